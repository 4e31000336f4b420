"""Each kernel alone against its plain reference, at sizes other than the engine's: widths and
vocabularies that are no power of two, head sizes in steps of 16, key/value groups, windows."""

import math

import numpy as np
import pytest
import torch

import helpers
import plain_gpt as P
from mini_gpt_inference_amd.ops import kernels

pytestmark = pytest.mark.gpu
DEV = "cuda"
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def rnd(gen, *shape, dtype="float32", scale=1.0):
    t = torch.randn(*shape, generator=gen, dtype=torch.float32) * scale
    return t.to(TDT[dtype])


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


# ----------------------------------------------------------------------------- embedding, norm
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("with_pos", [True, False])
def test_embed(dtype, with_pos):
    g = torch.Generator().manual_seed(0)
    tok, pos = rnd(g, 37, 80, dtype=dtype), rnd(g, 19, 80, dtype=dtype)
    ids, positions = [5, 36, 0, 5, 12, 7, 30], [0, 18, 3, 4, 4, 9, 1]
    x = torch.full((7, 80), float("nan"), device=DEV)
    kernels.embed(i32(ids), i32(positions), tok.to(DEV), pos.to(DEV) if with_pos else None, x, 7)
    want = tok.double()[ids] + (pos.double()[positions] if with_pos else 0)
    helpers.assert_close(x, want, "float32", "embed")     # the sum itself is float32 in both cases


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width,bias,eps", [(80, True, 1e-5), (1000, False, 1e-2), (48, True, 1e-6), (75, True, 1e-5),
                                            (1030, False, 1e-5), (1600, True, 1e-5), (512, True, 1e-5), (2052, True, 1e-5),
                                            (256, True, 1e-5), (768, False, 1e-5), (1024, True, 1e-5), (1280, True, 1e-5),
                                            (2048, False, 1e-5)])
def test_layer_norm(out_dtype, width, bias, eps):
    g = torch.Generator().manual_seed(1)
    x = rnd(g, 9, width, scale=3.0) + 2.0
    x[3] = 5.0 + 1e-3 * torch.randn(width, generator=g)     # an almost constant row: eps decides
    w, b = 1 + 0.1 * rnd(g, width), rnd(g, width) if bias else None
    out = torch.empty(9, width, dtype=TDT[out_dtype], device=DEV)
    kernels.layer_norm(x.to(DEV), w.to(DEV), b.to(DEV) if bias else None, out, 9, eps)
    want = P.plain_layer_norm(x.double(), w.double(), b.double() if bias else None, eps)
    helpers.assert_close(out, want, out_dtype, "layer_norm")
    rows = [8, 0, 3]
    out2 = torch.empty(3, width, dtype=TDT[out_dtype], device=DEV)
    kernels.layer_norm(x.to(DEV), w.to(DEV), b.to(DEV) if bias else None, out2, 3, eps, rows=i32(rows))
    helpers.assert_close(out2, want[rows], out_dtype, "layer_norm gather")


# ----------------------------------------------------------------------------- linear
def _linear_want(a, w, bias, epi, prev):
    y = P.plain_linear(a.double(), w.double(), None if bias is None else bias.double())
    if epi == kernels.EPI_GELU:
        y = P.plain_gelu_tanh(y)
    if epi == kernels.EPI_RESIDUAL:
        y = prev.double() + y
    return y


@pytest.mark.parametrize("epi", [kernels.EPI_NONE, kernels.EPI_GELU, kernels.EPI_RESIDUAL])
@pytest.mark.parametrize("a_dt,w_dt,o_dt", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16"),
                                            ("bfloat16", "bfloat16", "float32"), ("bfloat16", "float32", "bfloat16")])
def test_linear_generic(a_dt, w_dt, o_dt, epi):
    if epi == kernels.EPI_RESIDUAL and o_dt != "float32":
        pytest.skip("the residual stream is float32")
    g = torch.Generator().manual_seed(2)
    n, k, o = 70, 48, 203
    a, w, bias = rnd(g, n, k, dtype=a_dt), rnd(g, o, k, dtype=w_dt, scale=0.3), rnd(g, o)
    prev = rnd(g, n, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    kernels.linear_generic(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi)
    tol = "float32" if (a_dt, w_dt, o_dt) == ("float32",) * 3 else "bfloat16"
    helpers.assert_close(out, _linear_want(a, w, bias, epi, prev), tol, "linear_generic")


@pytest.mark.parametrize("n_few", [1, 7, 16, 17, 32])
@pytest.mark.parametrize("a_dt,w_dt,o_dt,epi", [("float32", "float32", "float32", kernels.EPI_NONE),
                                                ("float32", "float32", "float32", kernels.EPI_RESIDUAL),
                                                ("float32", "float32", "float32", kernels.EPI_GELU),
                                                ("bfloat16", "float32", "bfloat16", kernels.EPI_GELU),
                                                ("bfloat16", "bfloat16", "float32", kernels.EPI_NONE)])
def test_linear_generic_few_rows_and_many_agree_bit_for_bit(a_dt, w_dt, o_dt, epi, n_few):
    """Up to 32 rows go to a kernel with a workgroup per 16 x 16 outputs, more to 64 x 64 tiles: every
    element is the same chain of fused multiply-adds along k in both, so a row's result is the same
    bits whichever kernel its step's size chooses (a decode step against a prompt's step)."""
    g = torch.Generator().manual_seed(23)
    n, k, o = 50, 208, 137      # an inner size that is no multiple of the few-rows kernel's stage of 64
    a, w, bias = rnd(g, n, k, dtype=a_dt), rnd(g, o, k, dtype=w_dt), rnd(g, o)
    prev = rnd(g, n, o, dtype=o_dt)
    many = prev.clone().to(DEV)
    kernels.linear_generic(a.to(DEV), w.to(DEV), bias.to(DEV), many, n, epi)
    few = prev.clone().to(DEV)
    kernels.linear_generic(a.to(DEV), w.to(DEV), bias.to(DEV), few, n_few, epi)
    assert torch.equal(few[:n_few], many[:n_few])
    assert torch.equal(few[n_few:], prev[n_few:].to(DEV)), "rows beyond n_rows were written"
    helpers.assert_close(few[:n_few], _linear_want(a, w, bias, epi, prev)[:n_few],
                         "float32" if "bfloat16" not in (a_dt, w_dt, o_dt) else "bfloat16", "few rows")


@pytest.mark.parametrize("k", [1, 3, 36, 40, 75, 130])
@pytest.mark.parametrize("n", [5, 70])
@pytest.mark.parametrize("a_dt,w_dt,o_dt", [("float32", "float32", "float32"), ("bfloat16", "bfloat16", "bfloat16")])
def test_linear_generic_takes_any_inner_size(a_dt, w_dt, o_dt, n, k):
    """Inner sizes that are no multiple of the kernels' stages (16 and 64), few rows and many: the
    stage's tail is zeros, the row's result the same chain of multiply-adds."""
    g = torch.Generator().manual_seed(k)
    o = 37
    a, w, bias = rnd(g, n + 1, k, dtype=a_dt), rnd(g, o, k, dtype=w_dt), rnd(g, o)
    a[n] = float("nan")         # the row behind the last one is never read into a sum
    out = torch.full((n + 1, o), 7.0, dtype=TDT[o_dt], device=DEV)
    kernels.linear_generic(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_GELU)
    helpers.assert_close(out[:n], _linear_want(a[:n], w, bias, kernels.EPI_GELU, None), o_dt if o_dt == "bfloat16" else "float32",
                         f"inner size {k}")
    assert (out[n] == 7.0).all()


def test_linear_generic_refuses_tensors_off_the_gpu():
    a, w = torch.zeros(4, 40, device=DEV), torch.zeros(8, 40, device=DEV)
    with pytest.raises(kernels.KernelError, match="GPU"):
        kernels.linear_generic(a.cpu(), w, None, torch.zeros(4, 8, device=DEV), 4)


# general=False lets the kernel for a decode step's rows (at most 16, inner size a multiple of 32)
# take what it can; general=True keeps every case on the kernel for up to 64 rows
@pytest.mark.parametrize("general", [False, True])
@pytest.mark.parametrize("n,k,o", [(1, 64, 257), (8, 512, 1536), (17, 96, 503), (33, 80, 48), (64, 2048, 512), (40, 512, 1536), (24, 768, 48), (60, 96, 64), (50, 768, 1003),
                                   (5, 48, 16), (16, 160, 503), (12, 1600, 48), (7, 2048, 512), (3, 32, 20),
                                   (9, 768, 130)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
def test_linear_skinny(n, k, o, epi, o_dt, general):
    g = torch.Generator().manual_seed(3)
    a, w, bias = rnd(g, n + 2, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 2, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi, general_only=general)
    if not general and k % 32 == 0:
        # the same product from the packed copy of the matrix: the same sums in the same order
        packed = kernels.pack_weight(w.to(DEV))
        out_p = prev.clone().to(DEV)
        assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out_p, n, epi, w_packed=packed)
        assert torch.equal(out_p, out), "the packed matrix gives another result"
        # more than 16 rows: all rows in one workgroup per column tile, or 16 rows to a workgroup
        for mode in (kernels.ROWS_SHARE_W, kernels.ROWS_GROUPS):
            out_m = prev.clone().to(DEV)
            assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out_m, n, epi, w_packed=packed,
                                         rows_mode=mode)
            helpers.assert_close(out_m[:n], _linear_want(a, w, bias, epi, prev)[:n], "bfloat16", f"rows mode {mode}")
            assert torch.equal(out_m[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
        # 16, 8, 4 or 1 rows to a workgroup: the same sums whatever the groups
        outs = []
        for rpg in (16, 8, 1):
            out_g = prev.clone().to(DEV)
            assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out_g, n, epi, w_packed=packed,
                                         rows_mode=kernels.ROWS_GROUPS, rows_per_group=rpg)
            outs.append(out_g)
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), "the groups' size changes the result"
        helpers.assert_close(outs[2][:n], _linear_want(a, w, bias, epi, prev)[:n], "bfloat16", "groups of 1 row")
        assert torch.equal(outs[2][n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
    helpers.assert_close(out[:n], _linear_want(a, w, bias, epi, prev)[:n], "bfloat16", f"skinny {n}x{k}x{o}")
    assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
    out2 = prev.clone().to(DEV)
    assert kernels.linear_skinny(a.to(DEV), w.to(DEV), None, out2, n, epi, general_only=general)
    helpers.assert_close(out2[:n], _linear_want(a, w, None, epi, prev)[:n], "bfloat16", "skinny without bias")


@pytest.mark.parametrize("n,k,o", [(65, 64, 257), (300, 512, 1536), (129, 96, 503), (2048, 80, 48), (128, 2048, 128),
                                   (1000, 48, 130), (600, 1072, 136)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
def test_linear_mfma(n, k, o, epi, o_dt):
    g = torch.Generator().manual_seed(6)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi)
    helpers.assert_close(out, _linear_want(a, w, bias, epi, prev), "bfloat16", f"mfma {n}x{k}x{o}")
    # rows beyond n_rows are left alone
    out2 = prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), None, out2, n - 3, epi)
    assert torch.equal(out2[n - 3:], prev[n - 3:].to(DEV))
    helpers.assert_close(out2[:n - 3], _linear_want(a, w, None, epi, prev)[:n - 3], "bfloat16", "mfma partial rows")


@pytest.mark.parametrize("n,k,o", [(300, 80, 257), (513, 512, 520), (256, 2048, 256), (1000, 48, 130), (70, 64, 1030),
                                   (40, 1616, 272)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
@pytest.mark.parametrize("shape", [0, 1, 2, 3, 4, 5, 6, 7])
def test_linear_mfma_each_tile_shape(n, k, o, epi, o_dt, shape):
    """Each tile shape forced at sizes that cut its tiles everywhere: rows and columns past the end, an
    inner size that ends inside a step, several tiles each way.  Shapes 5 and 6: the 64 x 64 and 32 x 32
    tiles with four steps on their way from memory, in whole rounds of four (inner sizes of 1, 2, 8, 26
    and 32 steps: rounds that end beyond the last step).  Shape 7: the 64 x 64 tile with two wave groups,
    each one half of every step along k (also a last step of which only the first half exists); float32
    outputs only."""
    if shape == 7 and o_dt != "float32":
        a, w = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV), torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
        assert not kernels.linear_mfma(a, w, None, torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV), 64, epi, shape=7)
        return
    g = torch.Generator().manual_seed(16)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 2, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi, shape=shape)
    helpers.assert_close(out[:n], _linear_want(a, w, bias, epi, prev[:n]), "bfloat16", f"shape {shape} {n}x{k}x{o}")
    assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"


@pytest.mark.parametrize("n,k,o", [(300, 64, 257), (513, 512, 520), (256, 2048, 256), (1000, 128, 130), (130, 192, 400),
                                   (200, 320, 72), (40, 2112, 272)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
@pytest.mark.parametrize("shape", [8, 9, 10, 11, 12])
def test_linear_mfma_slices_straight_into_lds(n, k, o, epi, o_dt, shape):
    """The variants whose operand slices go from memory straight into LDS (tiles of 32 x 32 and 64 x 64 with
    four stages, 128 x 64 with three, 128 x 192 with two, 32 x 32 with six), forced at sizes that cut their tiles
    everywhere and at inner sizes of 1, 2, 3, 5, 8, 32 and 33 steps: fewer steps than stages, as many, and more."""
    g = torch.Generator().manual_seed(26)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 2, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi, shape=shape)
    helpers.assert_close(out[:n], _linear_want(a, w, bias, epi, prev[:n]), "bfloat16", f"shape {shape} {n}x{k}x{o}")
    assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"


def test_linear_mfma_straight_into_lds_wants_whole_steps():
    """An inner size that is no multiple of 64 is refused by those variants (nothing can be zeroed on its way
    into LDS), and the library's own choice then goes through registers."""
    g = torch.Generator().manual_seed(27)
    n, k, o = 256, 2064, 512
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    out = torch.zeros(n, o, device=DEV)
    for shape in (8, 9, 10, 11, 12):
        assert not kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_NONE, shape=shape)
    assert not kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_NONE, shape=13)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_NONE)
    helpers.assert_close(out, _linear_want(a, w, bias, kernels.EPI_NONE, None), "bfloat16", "through registers")


@pytest.mark.parametrize("n,k,o,shape", [(256, 2048, 512, 8), (2048, 2048, 512, 9), (2048, 3072, 768, 10), (8192, 512, 1536, 11),
                                         (1024, 3072, 768, 9), (2048, 1600, 4800, 11), (32, 1600, 4800, 12), (64, 1600, 6400, 8)])
def test_linear_mfma_chooses_the_variants_straight_into_lds(n, k, o, shape):
    """A long inner size (32 steps and more) with few tiles, a wide output under many rows, and few rows under
    a large matrix (the rows of a decode step; six stages while the tiles are at most 256): the library takes
    those variants by itself, so its result equals the forced one bit by bit."""
    g = torch.Generator().manual_seed(28)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n, o)
    out, out_f = prev.clone().to(DEV), prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_RESIDUAL)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out_f, n, kernels.EPI_RESIDUAL, shape=shape)
    assert torch.equal(out, out_f)
    helpers.assert_close(out, _linear_want(a, w, bias, kernels.EPI_RESIDUAL, prev), "bfloat16", "chosen")


@pytest.mark.parametrize("n,k,o,shape,parts", [(100, 2048, 96, 4, 4), (70, 1040, 132, 3, 2), (300, 6400, 64, 3, 8),
                                                (33, 576, 40, 4, 3), (130, 1600, 260, 2, 4), (64, 1600, 528, 6, 2),
                                                (50, 3200, 96, 5, 4), (48, 6400, 1600, None, 0), (90, 4128, 200, 7, 3),
                                                (100, 2048, 96, 8, 4), (300, 6400, 64, 9, 8), (130, 1600, 260, 10, 4),
                                                (140, 1088, 400, 11, 3), (64, 1600, 528, 12, 2)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
def test_linear_mfma_split_along_the_inner_size(n, k, o, shape, parts, epi, o_dt):
    """Several workgroups per tile, each with a stretch of the inner size (also one that ends inside a step
    and a number of stretches that leaves the last one short), their sums joined by the second kernel."""
    g = torch.Generator().manual_seed(18)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 2, o, dtype=o_dt)
    out = prev.clone().to(DEV)
    if shape is None:      # what the library chooses by itself: a split, 32 x 32 tiles, four steps in flight
        assert kernels.linear_mfma_partials(n, o, k, epi) > 0
        parts = kernels.linear_mfma_partials(n, o, k, epi) // (n * o)
    scratch = torch.full((parts * n * o + 8,), float("nan"), device=DEV)
    if shape is None:
        parts = None
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi, shape=shape, k_parts=parts,
                               partials=scratch)
    helpers.assert_close(out[:n], _linear_want(a, w, bias, epi, prev[:n]), "bfloat16", f"split {parts} of {k}")
    assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
    # twice the same: the sums are joined in a fixed order
    out2 = prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out2, n, epi, shape=shape, k_parts=parts,
                               partials=scratch)
    assert torch.equal(out, out2)
    # a buffer that is too small is refused when the split is forced, and not used when it is not
    if shape is not None:
        assert not kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out2, n, epi, shape=shape, k_parts=parts,
                                       partials=scratch[:16])


def test_linear_mfma_splits_by_itself_when_tiles_are_few_and_the_inner_size_long():
    g = torch.Generator().manual_seed(19)
    n, k, o = 140, 6416, 1600
    need = kernels.linear_mfma_partials(n, o, k, kernels.EPI_RESIDUAL)
    assert need > 0 and need % (n * o) == 0
    assert kernels.linear_mfma_partials(2048, 2048, 512, kernels.EPI_GELU) == 0
    # (an inner size of whole steps under 128 rows and more is not split even with the buffer there: it goes
    # straight into LDS, four steps deep; test_linear_mfma_chooses_the_variants_straight_into_lds)
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n, o)
    out, out1 = prev.clone().to(DEV), prev.clone().to(DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_RESIDUAL,
                               partials=torch.empty(need, device=DEV))
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out1, n, kernels.EPI_RESIDUAL)   # unsplit
    want = _linear_want(a, w, bias, kernels.EPI_RESIDUAL, prev)
    helpers.assert_close(out, want, "bfloat16", "split by itself")
    helpers.assert_close(out1, want, "bfloat16", "unsplit")
    assert not torch.equal(out, out1)      # another order of summation: it did split


def test_linear_mfma_chooses_the_largest_tiles_for_a_large_problem():
    """160 tiles of 256 x 256: the library takes that shape by itself, so the result equals the forced one bit by bit."""
    g = torch.Generator().manual_seed(17)
    n, k, o = 4096, 320, 2560
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    out, out_w = (torch.empty(n, o, dtype=torch.bfloat16, device=DEV) for _ in range(2))
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_GELU)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out_w, n, kernels.EPI_GELU, shape=0)
    assert torch.equal(out, out_w)
    helpers.assert_close(out, _linear_want(a, w, bias, kernels.EPI_GELU, None), "bfloat16", "large")


@pytest.mark.parametrize("general", [False, True])
@pytest.mark.parametrize("n,k,o,ln_bias,gather", [(8, 512, 1536, True, False), (3, 96, 503, False, True),
                                                  (40, 80, 257, True, True), (64, 2048, 64, False, False), (64, 512, 2048, True, False), (33, 768, 96, True, True),
                                                  (17, 1600, 48, True, False), (16, 1600, 130, True, True),
                                                  (1, 160, 48, False, False), (5, 768, 2050, True, True),
                                                  (2, 1024, 272, True, True), (4, 1600, 144, False, True), (7, 512, 80, True, True),
                                                  (1, 1600, 4800, True, True), (8, 2048, 96, True, True)])
def test_linear_skinny_through_a_folded_layer_norm(n, k, o, ln_bias, gather, general):
    g = torch.Generator().manual_seed(4)
    x = rnd(g, 70, k, scale=2.0) + 0.5
    x[:, 3] += 40.0                      # an outlier channel, as residual streams have
    lw, lb = 1 + 0.1 * rnd(g, k), rnd(g, k) if ln_bias else None
    w, bias = rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    rows = torch.randperm(70, generator=g)[:n].tolist() if gather else list(range(n))
    wf, colsum, bias_f = kernels.fold_layer_norm(w.to(DEV), lw.to(DEV), lb.to(DEV) if ln_bias else None, bias.to(DEV))
    # the fold itself: W' = W * gain, S = row sums of W', b' = b + W beta
    helpers.assert_close(wf, w.double() * lw.double(), "bfloat16", "folded matrix")
    helpers.assert_close(colsum, wf.double().sum(1), "float32", "column sums")
    helpers.assert_close(bias_f, bias.double() + (w.double() @ lb.double() if ln_bias else 0), "float32", "folded bias")
    out = torch.empty(n, o, dtype=torch.float32, device=DEV)
    assert kernels.linear_skinny(None, wf, bias_f, out, n, kernels.EPI_NONE, ln_x=x.to(DEV), ln_colsum=colsum,
                                 ln_eps=1e-5, ln_rows=i32(rows) if gather else None, general_only=general)
    if not general and k % 32 == 0:
        out_p = torch.empty_like(out)
        assert kernels.linear_skinny(None, wf, bias_f, out_p, n, kernels.EPI_NONE, ln_x=x.to(DEV), ln_colsum=colsum,
                                     ln_eps=1e-5, ln_rows=i32(rows) if gather else None,
                                     w_packed=kernels.pack_weight(wf))
        assert torch.equal(out_p, out), "the packed matrix gives another result"
    h = P.plain_layer_norm(x.double()[rows], lw.double(), lb.double() if ln_bias else None, 1e-5)
    helpers.assert_close(out, P.plain_linear(h, w.double(), bias.double()), "bfloat16", "LN + skinny")
    if not general and k % 32 == 0:
        for mode in (kernels.ROWS_SHARE_W, kernels.ROWS_GROUPS):
            out_m = torch.full((n + 1, o), float("nan"), dtype=torch.float32, device=DEV)
            assert kernels.linear_skinny(None, wf, bias_f, out_m, n, kernels.EPI_NONE, ln_x=x.to(DEV),
                                         ln_colsum=colsum, ln_eps=1e-5, ln_rows=i32(rows) if gather else None,
                                         rows_mode=mode)
            helpers.assert_close(out_m[:n], P.plain_linear(h, w.double(), bias.double()), "bfloat16",
                                 f"LN + skinny, rows mode {mode}")
            assert torch.isnan(out_m[n:]).all(), "rows beyond n_rows were written"
        for rpg in (16, 8, 4, 2, 1):
            out_g = torch.full((n + 1, o), float("nan"), dtype=torch.float32, device=DEV)
            assert kernels.linear_skinny(None, wf, bias_f, out_g, n, kernels.EPI_NONE, ln_x=x.to(DEV),
                                         ln_colsum=colsum, ln_eps=1e-5, ln_rows=i32(rows) if gather else None,
                                         rows_mode=kernels.ROWS_GROUPS, rows_per_group=rpg)
            # the rows' statistics are summed in an order that follows the rows of a workgroup,
            # so the results agree to rounding, not bit by bit
            helpers.assert_close(out_g[:n], P.plain_linear(h, w.double(), bias.double()), "bfloat16",
                                 f"LN + skinny, {rpg} rows to a workgroup")
            assert torch.isnan(out_g[n:]).all(), "rows beyond n_rows were written"


@pytest.mark.parametrize("general", [False, True])
@pytest.mark.parametrize("outlier", [None, 0, 7])
def test_folded_layer_norm_of_rows_far_from_zero(general, outlier):
    """Rows whose values lie 50 standard deviations from zero (and one channel further out still, also
    the first one): what the product rounds to bfloat16 must be the distance from a value of the
    row, not the value, or the rounding error of the offset drowns the row."""
    g = torch.Generator().manual_seed(40)
    n, k, o = 6, 256, 96
    x = rnd(g, n, k, scale=1.0) + torch.tensor([100.0, -100.0, 50.0, 0.0, 300.0, -75.0])[:, None]
    if outlier is not None:
        x[:, outlier] += 400.0
    lw, lb = 1 + 0.1 * rnd(g, k), rnd(g, k)
    w, bias = rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    wf, colsum, bias_f = kernels.fold_layer_norm(w.to(DEV), lw.to(DEV), lb.to(DEV), bias.to(DEV))
    out = torch.empty(n, o, dtype=torch.float32, device=DEV)
    assert kernels.linear_skinny(None, wf, bias_f, out, n, kernels.EPI_NONE, ln_x=x.to(DEV), ln_colsum=colsum,
                                 ln_eps=1e-5, general_only=general)
    h = P.plain_layer_norm(x.double(), lw.double(), lb.double(), 1e-5)
    helpers.assert_close(out, P.plain_linear(h, w.double(), bias.double()), "bfloat16", "LN of rows far from zero")


@pytest.mark.parametrize("general,n,rows_mode,rpg", [(False, 6, 0, 0), (True, 6, 0, 0), (True, 40, 0, 0),
                                                     (False, 40, kernels.ROWS_SHARE_W, 0),
                                                     (False, 40, kernels.ROWS_GROUPS, 0), (False, 64, kernels.ROWS_GROUPS, 0),
                                                     (False, 6, kernels.ROWS_GROUPS, 4), (False, 13, kernels.ROWS_GROUPS, 8),
                                                     (False, 40, kernels.ROWS_GROUPS, 4), (False, 16, 0, 0), (False, 7, kernels.ROWS_GROUPS, 1),
                                                     (False, 9, kernels.ROWS_GROUPS, 2)])
def test_linear_skinny_stores_keys_and_values(general, n, rows_mode, rpg):
    g = torch.Generator().manual_seed(5)
    k, h, hk, d, page, pages = 64, 4, 2, 16, 4, 23
    qw, kvw = h * d, hk * d
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, qw + 2 * kvw, k, dtype="bfloat16", scale=0.2), rnd(g, qw + 2 * kvw)
    kp = torch.full((pages, hk, page, d), float("nan"), dtype=torch.bfloat16, device=DEV)
    vp = kp.clone()
    slots = [4 * 8 + 3, 0, 7, -1, 4 * 2 + 1, 4 * 8 + 0]
    if n > 6:   # distinct slots all over the pool, a padded token now and then
        slots = torch.randperm(pages * page, generator=g)[:n].tolist()
        slots = [-1 if t % 9 == 4 else s for t, s in enumerate(slots)]
    out = torch.empty(n, qw + 2 * kvw, dtype=torch.bfloat16, device=DEV)
    assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.SK_EPI_QKV,
                                 scatter=(kp, vp, i32(slots), qw, kvw), general_only=general, rows_mode=rows_mode,
                                 rows_per_group=rpg)
    want = P.plain_linear(a.double(), w.double(), bias.double())
    helpers.assert_close(out, want, "bfloat16", "qkv")
    written = torch.zeros(pages * page, dtype=torch.bool)
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        written[slot] = True
        for head in range(hk):
            helpers.assert_close(kp[slot // page, head, slot % page], want[t, qw + head * d:qw + (head + 1) * d],
                                 "bfloat16", "stored key")
            helpers.assert_close(vp[slot // page, head, slot % page],
                                 want[t, qw + kvw + head * d:qw + kvw + (head + 1) * d], "bfloat16", "stored value")
    untouched = kp.float().cpu().permute(0, 2, 1, 3).reshape(pages * page, -1)[~written]
    assert torch.isnan(untouched).all(), "a slot that no token owns was written"


@pytest.mark.parametrize("n,k,o", [(64, 2048, 512), (40, 1024, 256), (17, 2048, 48), (33, 3072, 768), (24, 3072, 768)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_NONE, "float32"),
                                      (kernels.EPI_GELU, "bfloat16"), (kernels.EPI_RESIDUAL, "float32")])
def test_linear_skinny_with_the_inner_size_split_over_workgroups(n, k, o, epi, o_dt):
    """With scratch for the parts, a long inner size under more than 16 rows whose rows stay in one
    workgroup per column tile runs as two launches; the result is the unsplit kernel's up to the order
    of four sums.  Left to choose, the launcher splits only what it does not deal out in groups of
    16 rows (a small matrix with an inner size up to 2048)."""
    g = torch.Generator().manual_seed(16)
    need = 4 * n * o
    groups = kernels.linear_skinny_row_groups(n, o, k)
    assert groups == (o * k * 2 <= 6 << 20 if k <= 2048 else n > 32 and o * k * 2 <= 8 << 20)
    assert kernels.linear_skinny_partials(n, o, k, False, epi) == (0 if groups else need)
    # up to 16 rows: split only from an inner size of 3072 on
    assert kernels.linear_skinny_partials(16, o, k, False, epi) == (4 * 16 * o if k >= 3072 else 0)
    assert kernels.linear_skinny_partials(n, o, 512, False, epi) == 0         # a short inner size
    assert kernels.linear_skinny_partials(n, o, k, True, epi) == 0            # not through a folded LayerNorm
    a, w, bias = rnd(g, n + 2, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 2, o, dtype=o_dt)
    partials = torch.full((need,), float("nan"), device=DEV)
    for b in (bias, None):
        out = prev.clone().to(DEV)
        assert kernels.linear_skinny(a.to(DEV), w.to(DEV), None if b is None else b.to(DEV), out, n, epi,
                                     partials=partials, rows_mode=kernels.ROWS_SHARE_W)
        assert not torch.isnan(partials[:need]).any(), "the parts were not written: no split happened"
        partials.fill_(float("nan"))
        helpers.assert_close(out[:n], _linear_want(a, w, b, epi, prev)[:n], "bfloat16", f"split {n}x{k}x{o}")
        assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
    # too little scratch: the unsplit kernel, same result
    out2 = prev.clone().to(DEV)
    assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out2, n, epi, partials=partials[:need // 2],
                                 rows_mode=kernels.ROWS_SHARE_W)
    assert torch.isnan(partials).all(), "too little scratch was written to"
    helpers.assert_close(out2[:n], _linear_want(a, w, bias, epi, prev)[:n], "bfloat16", "unsplit")


@pytest.mark.parametrize("n,k,o", [(1, 3072, 768), (8, 6400, 1600), (16, 3072, 48), (3, 4096, 512)])
@pytest.mark.parametrize("epi,o_dt", [(kernels.EPI_NONE, "bfloat16"), (kernels.EPI_GELU, "bfloat16"),
                                      (kernels.EPI_RESIDUAL, "float32")])
def test_linear_skinny_few_rows_with_a_long_inner_size_split_over_workgroups(n, k, o, epi, o_dt):
    """Up to 16 rows under an inner size of 3072 and more and few column tiles: four workgroups per
    tile take a quarter of the inner size each when the caller brings scratch, one takes it all
    without; both against the plain product."""
    g = torch.Generator().manual_seed(61)
    need = kernels.linear_skinny_partials(n, o, k, False, epi)
    assert need == 4 * n * o
    assert kernels.linear_skinny_partials(n, o, 2048, False, epi) == 0       # not worth a second kernel
    assert kernels.linear_skinny_partials(n, 2048, k, False, epi) == 0       # column tiles enough
    a, w, bias = rnd(g, n + 1, k, dtype="bfloat16"), rnd(g, o, k, dtype="bfloat16", scale=k ** -0.5), rnd(g, o)
    prev = rnd(g, n + 1, o, dtype=o_dt)
    want = _linear_want(a, w, bias, epi, prev)
    partials = torch.full((need,), float("nan"), device=DEV)
    packed = kernels.pack_weight(w.to(DEV))
    for wp in (None, packed):
        out = prev.clone().to(DEV)
        assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, epi, partials=partials, w_packed=wp)
        assert not torch.isnan(partials).any(), "the parts were not written: no split happened"
        partials.fill_(float("nan"))
        helpers.assert_close(out[:n], want[:n], "bfloat16", f"few rows split {n}x{k}x{o}")
        assert torch.equal(out[n:], prev[n:].to(DEV)), "rows beyond n_rows were written"
    whole = prev.clone().to(DEV)
    assert kernels.linear_skinny(a.to(DEV), w.to(DEV), bias.to(DEV), whole, n, epi)
    helpers.assert_close(whole[:n], want[:n], "bfloat16", "unsplit")


@pytest.mark.parametrize("n,shape,k", [(70, None, 96), (300, 3, 96), (1100, 2, 96), (300, 1, 96), (520, 0, 96),
                                       (40, None, 832), (60, 6, 96), (33, 5, 1024), (200, 8, 256), (300, 9, 128),
                                       (520, 10, 192), (1100, 11, 64), (60, 12, 832)])
def test_linear_mfma_stores_keys_and_values(n, shape, k):
    """The tiled kernel's fused QKV product: the tile shape chosen by the size and each larger one forced
    (at 40 rows over 13 steps the library takes the variant with four steps in flight by itself);
    groups of heads; padded rows (slot -1) leave the pools alone."""
    g = torch.Generator().manual_seed(15)
    h, hk, d, page = 6, 2, 16, 8
    pages = n // page + 3
    qw, kvw = h * d, hk * d
    a, w, bias = rnd(g, n, k, dtype="bfloat16"), rnd(g, qw + 2 * kvw, k, dtype="bfloat16", scale=0.2), rnd(g, qw + 2 * kvw)
    kp = torch.full((pages, hk, page, d), float("nan"), dtype=torch.bfloat16, device=DEV)
    vp = kp.clone()
    slots = torch.randperm(pages * page, generator=g)[:n].tolist()
    for t in range(0, n, 7):
        slots[t] = -1
    out = torch.empty(n, qw + 2 * kvw, dtype=torch.bfloat16, device=DEV)
    assert kernels.linear_mfma(a.to(DEV), w.to(DEV), bias.to(DEV), out, n, kernels.EPI_NONE,
                               scatter=(kp, vp, i32(slots), qw, kvw), shape=shape)
    want = P.plain_linear(a.double(), w.double(), bias.double())
    helpers.assert_close(out, want, "bfloat16", "qkv")
    kflat = kp.float().cpu().permute(0, 2, 1, 3).reshape(pages * page, kvw)
    vflat = vp.float().cpu().permute(0, 2, 1, 3).reshape(pages * page, kvw)
    live = torch.tensor([s for s in slots if s >= 0])
    rows = torch.tensor([t for t, s in enumerate(slots) if s >= 0])
    helpers.assert_close(kflat[live], want[rows, qw:qw + kvw], "bfloat16", "stored keys")
    helpers.assert_close(vflat[live], want[rows, qw + kvw:], "bfloat16", "stored values")
    untouched = torch.ones(pages * page, dtype=torch.bool)
    untouched[live] = False
    assert torch.isnan(kflat[untouched]).all() and torch.isnan(vflat[untouched]).all()


def test_linear_skinny_refuses_what_it_cannot_do():
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    a = torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV)
    assert not kernels.linear_skinny(a, w, None, torch.zeros(65, 32, dtype=torch.bfloat16, device=DEV), 65)
    assert not kernels.linear_skinny(a.float(), w, None, torch.zeros(65, 32, dtype=torch.bfloat16, device=DEV), 4)


# ----------------------------------------------------------------------------- cache write and attention
class PagedCase:
    """Random requests with part of their tokens already cached, laid out in scattered pages."""

    def __init__(self, seq_lens, q_lens, h, hk, d, page, dtype, seed=0, poison=True, spikes=()):
        """spikes: (request, query index within the step, key position, head): that query and that key
        are made long and parallel, so that this one score stands out among hundreds and the query's
        output is that key's value; a kernel that misses the key, or takes another for it, shows."""
        g = torch.Generator().manual_seed(seed)
        self.h, self.hk, self.d, self.page = h, hk, d, page
        self.seq_lens, self.q_lens = seq_lens, q_lens
        n_pages = sum(-(-s // page) for s in seq_lens) + 3
        order = torch.randperm(n_pages, generator=g).tolist()
        self.k = [rnd(g, s, hk, d, dtype=dtype) for s in seq_lens]
        self.v = [rnd(g, s, hk, d, dtype=dtype) for s in seq_lens]
        self.q = [rnd(g, ql, h, d, dtype=dtype) for ql in q_lens]
        for r, qi, key, head in spikes:
            assert key <= seq_lens[r] - q_lens[r] + qi, "a query sees no later key"
            u = torch.randn(d, generator=g)
            u = (3.0 * math.sqrt(d) * u / u.norm()).to(TDT[dtype])      # |u|^2 = 9 d: the score is 9 d * scale
            self.q[r][qi, head] = u
            self.k[r][key, head // (h // hk)] = u
        fill = float("nan") if poison else 0.0
        kp = torch.full((n_pages, hk, page, d), fill, dtype=TDT[dtype])
        vp = kp.clone()
        mb = max(-(-s // page) for s in seq_lens) + 1
        bt = torch.full((len(seq_lens), mb), -1, dtype=torch.int32)
        self.slots = []
        for r, s in enumerate(seq_lens):
            for b in range(-(-s // page)):
                bt[r, b] = order.pop()
            for t in range(s):
                pg, off = bt[r, t // page].item(), t % page
                kp[pg, :, off] = self.k[r][t]
                vp[pg, :, off] = self.v[r][t]
            self.slots += [bt[r, t // page].item() * page + t % page for t in range(s - q_lens[r], s)]
        self.kp, self.vp, self.bt = kp.to(DEV), vp.to(DEV), bt.to(DEV)
        self.n = sum(q_lens)
        self.cu = i32(np.concatenate([[0], np.cumsum(q_lens)]))
        self.sl = i32(seq_lens)
        self.q_req = i32([r for r, ql in enumerate(q_lens) for _ in range(ql)])
        self.q_flat = torch.cat([q.reshape(-1, h * d) for q in self.q]).to(DEV)

    def want(self, scale, window):
        outs = []
        for r, (s, ql) in enumerate(zip(self.seq_lens, self.q_lens)):
            # the plain attention over the whole sequence; the step's queries are its last q_len rows
            qfull = torch.zeros(self.h, s, self.d, dtype=P.DT)
            qfull[:, s - ql:] = self.q[r].double().transpose(0, 1)
            o = P.plain_causal_attention(qfull, self.k[r].double().transpose(0, 1),
                                         self.v[r].double().transpose(0, 1), scale=scale, window=window)
            outs.append(o[s - ql:])
        return torch.cat(outs)


ATTENTION_CASES = [
    # the reference's own cases (tests/test_triton.py:83-154): uniform, ragged around a page, one key
    dict(seq_lens=[16] * 4, q_lens=[1] * 4, h=4, hk=4, d=64, page=8),
    dict(seq_lens=[3, 8, 9, 17, 24], q_lens=[1] * 5, h=4, hk=4, d=64, page=8),
    dict(seq_lens=[1, 1], q_lens=[1, 1], h=2, hk=2, d=64, page=8),
    # other sizes: groups, head sizes in steps of 16, portions, pages of other sizes, long contexts
    dict(seq_lens=[40, 7, 130], q_lens=[5, 7, 2], h=6, hk=2, d=48, page=4),
    dict(seq_lens=[300, 65], q_lens=[1, 33], h=3, hk=1, d=16, page=16),
    dict(seq_lens=[77, 200], q_lens=[77, 1], h=2, hk=2, d=128, page=32),
    dict(seq_lens=[129], q_lens=[64], h=5, hk=5, d=80, page=16),
    dict(seq_lens=[333, 70, 200], q_lens=[333, 3, 130], h=4, hk=2, d=32, page=16),
    dict(seq_lens=[500], q_lens=[190], h=2, hk=1, d=96, page=8),
]


@pytest.mark.parametrize("window", [0, 5, 70])
@pytest.mark.parametrize("case", range(len(ATTENTION_CASES)))
@pytest.mark.parametrize("kernel", ["generic-float32", "generic-bfloat16", "split-bfloat16", "splitfast-bfloat16",
                                    "prefill-bfloat16"])
def test_paged_attention(kernel, case, window):
    name, dtype = kernel.split("-")
    c = PagedCase(**ATTENTION_CASES[case], dtype=dtype, seed=case)
    scale = 0.37 if case % 2 else 1.0 / math.sqrt(c.d)
    out = torch.full((c.n, c.h * c.d), float("nan"), dtype=TDT[dtype], device=DEV)
    args = (c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, c.q_req, c.n, len(c.seq_lens), c.h, scale, window)
    if name == "generic":
        kernels.paged_attention_generic(*args, fast_exp=dtype == "bfloat16")
    elif name == "prefill":
        if c.d not in (32, 64, 96, 128):
            pytest.skip("the MFMA tile kernel takes head sizes 32, 64, 96, 128")
        assert kernels.prefill_attention_bf16(c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, len(c.seq_lens),
                                              max(c.q_lens), c.h, scale, window)
    else:
        if name == "splitfast" and c.d not in (16, 32, 64, 128):
            pytest.skip("the wide-load variant takes head sizes 16, 32, 64, 128")
        assert kernels.paged_attention_split_bf16(*args, fast=name == "splitfast")
    helpers.assert_close(out, c.want(scale, window), dtype, f"{kernel} case {case} window {window}")


@pytest.mark.parametrize("window", [0, 33])
@pytest.mark.parametrize("d", [32, 64])
def test_prefill_attention_with_many_tiles(d, window):
    """More than 320 query tiles in the step: the tile kernel then runs with one wave group and two
    workgroups on a compute unit instead of two wave groups that split the keys."""
    lens = [130 + 7 * i for i in range(11)]
    c = PagedCase(seq_lens=lens, q_lens=[70 + (i % 3) for i in range(11)], h=16, hk=4, d=d, page=16,
                  dtype="bfloat16", seed=d)
    assert 11 * 2 * 16 > 320
    out = torch.full((c.n, c.h * c.d), float("nan"), dtype=torch.bfloat16, device=DEV)
    scale = 1.0 / math.sqrt(d)
    assert kernels.prefill_attention_bf16(c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, len(lens), max(c.q_lens),
                                          c.h, scale, window)
    helpers.assert_close(out, c.want(scale, window), "bfloat16", f"many tiles, head size {d}")


LONG_PREFILL_CASES = {
    # the benchmarked prefill step: two whole prompts of 1,024 tokens, 8 heads of 64 (256 query tiles:
    # two wave groups split every 256 keys), and the same with more than 320 tiles (one wave group)
    "2x1024-d64": dict(seq_lens=[1024, 1024], q_lens=[1024, 1024], h=8, hk=8, d=64, page=16),
    "3x1024-d64": dict(seq_lens=[1024, 1000, 1024], q_lens=[1024, 1000, 1024], h=8, hk=8, d=64, page=16),
    "1x1024-d128": dict(seq_lens=[1024], q_lens=[1024], h=4, hk=4, d=128, page=16),
    "6x1024-d128": dict(seq_lens=[1024] * 6, q_lens=[1024] * 6, h=4, hk=2, d=128, page=32),
    # portions of 64 to 512 tokens over 512 and 900 cached keys, few tiles and many
    "portions-d64": dict(seq_lens=[576, 1024, 1024, 964], q_lens=[64, 124, 512, 64], h=8, hk=8, d=64, page=16),
    "portions-d64-many": dict(seq_lens=[576, 1024, 1024, 964], q_lens=[64, 124, 512, 64], h=32, hk=8, d=64, page=16),
    "portions-d128": dict(seq_lens=[1024, 612, 1000], q_lens=[512, 100, 100], h=4, hk=4, d=128, page=8),
    "portions-d128-many": dict(seq_lens=[1024, 612, 1000], q_lens=[512, 100, 100], h=32, hk=4, d=128, page=8),
}


@pytest.mark.parametrize("name", sorted(LONG_PREFILL_CASES))
def test_prefill_attention_at_the_benchmarked_lengths(name):
    """The MFMA tile kernel with whole prompts of 1,024 tokens and with portions over 512 and 900
    cached keys, head sizes 64 and 128, in both of its modes (two wave groups that split every 256
    keys while the step has at most 320 query tiles, one wave group beyond), pages scattered over a
    NaN-poisoned pool.  Random scores alone are nearly flat over so many keys: in every request a
    few queries get one key that stands out (the first key, one a few blocks back, the last key of a
    128-key block, the query's own), and the query's output must be that key's value."""
    spec = LONG_PREFILL_CASES[name]
    tiles = sum(-(-q // 64) for q in spec["q_lens"]) * spec["h"]
    assert (tiles > 320) == (name.startswith(("3x", "6x")) or name.endswith("many")), tiles
    spikes = []
    for r, (s, ql) in enumerate(zip(spec["seq_lens"], spec["q_lens"])):
        first = s - ql
        for j, (qi, key) in enumerate([(ql - 1, 0), (ql - 1 - 7, max(first + ql - 8 - 300, 1)), (ql // 2, 127),
                                       (ql // 3, first + ql // 3), (1, first + 1), (ql - 2, 383)]):
            if key <= first + qi:
                spikes.append((r, qi, key, (r + j) % spec["h"]))
    assert len({(r, key) for r, _, key, _ in spikes}) == len({(r, qi) for r, qi, _, _ in spikes}) == len(spikes)
    c = PagedCase(**spec, dtype="bfloat16", seed=len(name), spikes=spikes)
    scale = 1.0 / math.sqrt(c.d)
    out = torch.full((c.n, c.h * c.d), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert kernels.prefill_attention_bf16(c.q_flat, out, c.kp, c.vp, c.bt, c.cu, c.sl, len(c.seq_lens),
                                          max(c.q_lens), c.h, scale, 0)
    want = c.want(scale, 0)
    helpers.assert_close(out, want, "bfloat16", name)
    # the spiked queries really are decided by one key (so the comparison above pins the lookup)
    offs = np.concatenate([[0], np.cumsum(c.q_lens)])
    for r, qi, key, head in spikes:
        row = want[offs[r] + qi, head * c.d:(head + 1) * c.d]
        helpers.assert_close(row, c.v[r][key, head // (c.h // c.hk)].double(), "bfloat16", f"{name}: spike {r, qi, key}")


@pytest.mark.parametrize("window", [0, 20])
def test_single_tokens_and_portions_told_apart_on_the_device(window):
    """What a padded graph of a step with prompt portions launches: the decode kernel over the first 16
    tokens, leaving out those of requests with several tokens; the tile kernel over all requests
    (padded to 8, the padding bringing no tokens), leaving out the single tokens among the first 16.
    Together they write every token's row once: single tokens before and after the 16th, portions
    that start before it."""
    q_lens = [1, 1, 1, 9, 1, 1, 30]            # tokens 0, 1, 2 | 3..11 | 12 | 13 | 14..43: token 13 < 16 <= 14 + 30
    seq_lens = [50, 1, 77, 40, 200, 18, 64]
    c = PagedCase(seq_lens=seq_lens, q_lens=q_lens, h=4, hk=2, d=64, page=16, dtype="bfloat16", seed=3)
    scale = 0.125
    r_cap, n_cap = 8, 48
    cu = torch.full((r_cap + 1,), c.n, dtype=torch.int32)
    cu[:len(q_lens) + 1] = c.cu.cpu()
    sl = torch.zeros(r_cap, dtype=torch.int32)
    sl[:len(q_lens)] = c.sl.cpu()
    bt = torch.full((r_cap, c.bt.shape[1]), -1, dtype=torch.int32)
    bt[:len(q_lens)] = c.bt.cpu()
    q_req = torch.full((n_cap,), -1, dtype=torch.int32)
    q_req[:c.n] = c.q_req.cpu()
    pos = torch.zeros(n_cap, dtype=torch.int32)
    pos[:c.n] = torch.tensor([s - ql + j for s, ql in zip(seq_lens, q_lens) for j in range(ql)], dtype=torch.int32)
    qp = torch.zeros(n_cap, c.q_flat.shape[1], dtype=torch.bfloat16, device=DEV)
    qp[:c.n] = c.q_flat
    out = torch.full((n_cap, c.h * c.d), float("nan"), dtype=torch.bfloat16, device=DEV)
    cu, sl, bt, q_req, pos = (t.to(DEV) for t in (cu, sl, bt, q_req, pos))
    assert kernels.paged_attention_decode_bf16(qp, out, c.kp, c.vp, bt, pos, q_req, 16, c.h, scale, window, cu_q=cu)
    singles = [0, 1, 2, 12, 13]
    others = [t for t in range(c.n) if t not in singles]
    assert torch.isnan(out[others].float()).all(), "the decode kernel wrote a portion's token"
    assert not torch.isnan(out[singles].float()).any()
    assert kernels.prefill_attention_bf16(qp, out, c.kp, c.vp, bt, cu, sl, r_cap, n_cap, c.h, scale, window,
                                          single_below=16)
    helpers.assert_close(out[:c.n], c.want(scale, window), "bfloat16", "single tokens and portions together")
    assert torch.isnan(out[c.n:].float()).all(), "a padded row was written"


DECODE_CASES = [
    dict(seq_lens=[600, 1, 64, 65, 513, 300], q_lens=[1] * 6, h=4, hk=2, d=64, page=16),
    dict(seq_lens=[130, 1030, 7], q_lens=[1] * 3, h=3, hk=3, d=128, page=32),
    dict(seq_lens=[257, 31, 512, 511], q_lens=[1] * 4, h=6, hk=2, d=32, page=8),
    dict(seq_lens=[90, 700], q_lens=[1] * 2, h=2, hk=1, d=16, page=4),
    dict(seq_lens=[100, 550, 13], q_lens=[1] * 3, h=2, hk=2, d=64, page=12),   # a page size that is no power of two
]


@pytest.mark.parametrize("window", [0, 5, 70])
@pytest.mark.parametrize("case", range(len(ATTENTION_CASES) + len(DECODE_CASES)))
def test_paged_attention_decode(case, window):
    """The decode step's kernel: by position and block table row, for any token; with identity=True
    where every request brings one token.  Unused block table entries hold numbers far outside the
    pool, and a padded token leaves its output row alone."""
    spec = (ATTENTION_CASES + DECODE_CASES)[case]
    if spec["d"] not in (16, 32, 64, 128):
        pytest.skip("head sizes 16, 32, 64, 128")
    c = PagedCase(**spec, dtype="bfloat16", seed=case)
    scale = 0.37 if case % 2 else 1.0 / math.sqrt(c.d)
    bt = c.bt.clone()
    bt[bt < 0] = 10 ** 6
    positions = i32([p for s, ql in zip(c.seq_lens, c.q_lens) for p in range(s - ql, s)] + [0])
    q_req = torch.cat([c.q_req, i32([-1])])
    q = torch.cat([c.q_flat, c.q_flat[:1]])
    want = c.want(scale, window)
    modes = [False, True] if all(ql == 1 for ql in c.q_lens) else [False]
    for identity in modes:
        out = torch.full((c.n + 1, c.h * c.d), 7.0, dtype=torch.bfloat16, device=DEV)
        if identity:   # the padded token's row of the block table exists, as in a padded step
            bt_i = torch.cat([bt, torch.full_like(bt[:1], 10 ** 6)])
        else:
            bt_i = bt
        took = kernels.paged_attention_decode_bf16(q, out, c.kp, c.vp, bt_i, positions, q_req, c.n + 1, c.h, scale,
                                                   window, identity=identity)
        if c.page & (c.page - 1):
            assert not took, "page sizes that are no power of two go to the general kernels"
            return
        assert took
        helpers.assert_close(out[:c.n], want, "bfloat16", f"decode case {case} window {window} identity {identity}")
        assert (out[c.n] == 7.0).all(), "a padded token's row was written"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_kv_write_and_padding(dtype):
    g = torch.Generator().manual_seed(7)
    n, hk, d, page, pages = 5, 3, 16, 4, 6
    qkv = rnd(g, n, 7 + 2 * hk * d, dtype=dtype).to(DEV)
    kp = torch.full((pages, hk, page, d), float("nan"), dtype=TDT[dtype], device=DEV)
    vp = kp.clone()
    slots = [9, 0, -1, 23, 10]
    kernels.kv_write(qkv, 7, 7 + hk * d, kp, vp, i32(slots), n)
    for t, s in enumerate(slots):
        if s < 0:
            continue
        assert torch.equal(kp[s // page, :, s % page].reshape(-1), qkv[t, 7:7 + hk * d])
        assert torch.equal(vp[s // page, :, s % page].reshape(-1), qkv[t, 7 + hk * d:])
    assert torch.isnan(kp.float()).sum().item() == (pages * page - 4) * hk * d
    # a padded token (q_req = -1) is skipped by attention: its output row is left alone
    c = PagedCase(seq_lens=[9], q_lens=[2], h=3, hk=3, d=16, page=4, dtype=dtype)
    out = torch.full((3, 48), 7.0, dtype=TDT[dtype], device=DEV)
    q = torch.cat([c.q_flat, c.q_flat[:1]])
    kernels.paged_attention_generic(q, out, c.kp, c.vp, c.bt, c.cu, c.sl, i32([0, 0, -1]), 3, 1, 3, 0.25, 0)
    assert (out[2] == 7.0).all() and torch.isfinite(out[:2].float()).all()


# ----------------------------------------------------------------------------- sampling
def _sample(logits, temperature, top_k=None, top_p=None, seeds=None, idx=None, engine_seed=0, real_vocab=None):
    m, v = logits.shape
    out = torch.full((m,), -1, dtype=torch.int32, device=DEV)
    kernels.sample(logits.to(DEV), m, real_vocab or v, torch.tensor(temperature, dtype=torch.float32, device=DEV),
                   None if top_k is None else i32(top_k),
                   None if top_p is None else torch.tensor(top_p, dtype=torch.float32, device=DEV),
                   None if seeds is None else torch.tensor(seeds, dtype=torch.int64, device=DEV),
                   None if idx is None else i32(idx), engine_seed, out)
    return out.cpu().tolist()


def test_greedy_is_argmax_with_the_lowest_index_on_ties_and_respects_the_vocabulary_mask():
    g = torch.Generator().manual_seed(8)
    logits = rnd(g, 6, 50304)
    logits[1, 777] = logits[1, 40000] = 50.0
    logits[2, 50300] = 99.0                       # beyond the real vocabulary
    got = _sample(logits, [0.0] * 6, real_vocab=50257)
    want = [P.plain_sample(row.numpy(), 0.0, None, None, 0.0, 50257)[0] for row in logits]
    assert got == want and got[1] == 777 and got[2] < 50257


def test_greedy_ties_at_every_distance_and_rows_that_are_not_aligned():
    """Equal maxima in one vector of four, in one thread's vectors, in different waves; the last id that
    may be chosen; a vocabulary that leaves rows unaligned and a tail of one to three logits."""
    g = torch.Generator().manual_seed(12)
    for rows, vocab, real in ((6, 50304, 50257), (3, 50257, 50257), (7, 9003, 9001), (3, 300, 300)):
        logits = rnd(g, rows, vocab)
        logits[0, real - 5] = logits[0, 11] = 60.0
        logits[1, real - 1] = 70.0
        far = 4096 + 5 if real > 4101 else 200
        logits[-1, 5] = logits[-1, 6] = logits[-1, far] = 65.0
        got = _sample(logits, [0.0] * rows, real_vocab=real)
        want = [P.plain_sample(row.numpy(), 0.0, None, None, 0.0, real)[0] for row in logits]
        assert got == want and got[0] == 11 and got[1] == real - 1 and got[-1] == 5


@pytest.mark.parametrize("rows,n_out,k_dim,limit,packed,bias", [(1, 1008, 96, 1001, True, False), (5, 50304, 512, 50257, True, False),
                                                             (16, 208, 64, 208, False, True), (8, 4096, 1600, 4090, True, True),
                                                             (3, 2000, 768, 1999, False, False)])
def test_head_leaves_the_best_column_of_every_tile_and_greedy_rows_choose_from_them(rows, n_out, k_dim, limit, packed, bias):
    """The logits are those of the plain product; every tile's best is the plain argmax over the
    tile's columns below the limit (the lowest column among equals: two rows of the matrix are the
    same, inside a tile and across tiles); and greedy rows that read the tiles' bests choose what
    they choose from the logits themselves, beside seeded rows that still read the logits."""
    g = torch.Generator().manual_seed(rows * 7 + n_out)
    a = rnd(g, rows, k_dim, dtype="bfloat16")
    w = rnd(g, n_out, k_dim, dtype="bfloat16", scale=0.1)
    w[17] = w[21]                          # equal logits within a tile
    w[n_out - 40] = w[3]                   # and in two tiles far apart
    a[0] = (w[3].float() * 8).bfloat16()   # row 0 points at them: its largest logits are the equal pair
    if rows > 1:
        a[-1] = (w[n_out - 1].float() * 8).bfloat16()   # the last row's largest logit lies past the limit (if limit < n_out)
    b = rnd(g, n_out, scale=0.1) if bias else None
    if bias:
        b[17], b[n_out - 40] = b[21], b[3]
    out = torch.full((rows, n_out), float("nan"), device=DEV)
    tiles = n_out // 16
    bv = torch.full((rows + 2, tiles), float("nan"), device=DEV)
    bi = torch.full((rows + 2, tiles), -3, dtype=torch.int32, device=DEV)
    wd = w.to(DEV)
    assert kernels.linear_head_best(a.to(DEV), wd, None if b is None else b.to(DEV), out, rows, bv, bi, limit,
                                    w_packed=kernels.pack_weight(wd) if packed else None)
    want = _linear_want(a, w, b, kernels.EPI_NONE, None)
    helpers.assert_close(out, want, "bfloat16", "head")
    # the tiles' bests are exact statements about the logits that were stored
    got = out.cpu()
    masked = got.clone()
    masked[:, limit:] = -float("inf")
    per_tile = masked.view(rows, tiles, 16)
    want_val, want_off = per_tile.max(dim=2)
    first = (per_tile == want_val.unsqueeze(2)).int().argmax(dim=2)     # the lowest column among equals
    want_idx = first + 16 * torch.arange(tiles).unsqueeze(0)
    live = torch.isfinite(want_val)       # a tile wholly past the limit holds -inf and no column
    assert torch.equal(bv[:rows].cpu()[live], want_val[live])
    assert torch.equal(bi[:rows].cpu()[live].long(), want_idx[live])
    assert (bv[:rows].cpu()[~live] == -float("inf")).all()
    assert torch.isnan(bv[rows:]).all() and (bi[rows:] == -3).all()
    # choosing from them
    temps = [0.0] * rows
    if rows > 2:
        temps[1] = 0.8
    tk = torch.tensor(temps, device=DEV)
    seeds = torch.arange(rows, dtype=torch.int64, device=DEV)
    idx = torch.zeros(rows, dtype=torch.int32, device=DEV)
    from_logits = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    from_tiles = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    kernels.sample(out, rows, limit, tk, None, None, seeds, idx, 5, from_logits)
    kernels.sample(out, rows, limit, tk, None, None, seeds, idx, 5, from_tiles, tile_best=(bv, bi))
    assert torch.equal(from_logits, from_tiles)
    plain = [P.plain_sample(got[r].numpy(), 0.0, None, None, 0.0, limit)[0] for r in range(rows) if temps[r] == 0.0]
    assert [t for t, temp in zip(from_tiles.cpu().tolist(), temps) if temp == 0.0] == plain
    assert from_tiles[0].item() == 3 and from_tiles[-1].item() < limit


def test_head_with_tile_bests_refuses_what_its_kernel_does_not_take():
    g = torch.Generator().manual_seed(4)
    for rows, n_out, k_dim in ((17, 208, 64), (4, 200, 64), (4, 208, 48)):
        a, w = rnd(g, rows, k_dim, dtype="bfloat16").to(DEV), rnd(g, n_out, k_dim, dtype="bfloat16").to(DEV)
        out = torch.zeros(rows, n_out, device=DEV)
        tiles = max(n_out // 16, 1)
        bv, bi = torch.zeros(rows, tiles, device=DEV), torch.zeros(rows, tiles, dtype=torch.int32, device=DEV)
        assert not kernels.linear_head_best(a, w, None, out, rows, bv, bi, n_out)
        assert (out == 0).all()


def test_sampling_prepares_the_next_decode_step_on_the_device():
    """Greedy and seeded rows; two cache groups with pages of 4 and 8 slots; a padded row is left alone;
    a position past the block table's end gets slot -1."""
    g = torch.Generator().manual_seed(21)
    rows, vocab, n_stride, r_stride, max_blocks = 5, 300, 8, 6, 4
    page_sizes = [4, 8]
    positions = [3, 7, 0, 15, 9]
    q_req = [0, 1, -1, 3, 4]
    bt = torch.randint(0, 50, (2, r_stride, max_blocks), generator=g, dtype=torch.int32)
    bt[0, 1, 2] = -1                     # request 1 has no page yet for position 8 in group 0
    tok0 = torch.randint(0, vocab, (n_stride,), generator=g, dtype=torch.int32)
    d = dict(token_ids=tok0.clone().to(DEV), positions=i32(positions + [0] * 3),
             seq_lens=i32([p + 1 for p in positions] + [0]), q_req=i32(q_req + [-1] * 3),
             slot_mapping=torch.full((2, n_stride), -7, dtype=torch.int32, device=DEV), block_tables=bt.to(DEV),
             page_sizes=i32(page_sizes), history=torch.full((3, 6), -5, dtype=torch.int32, device=DEV),
             history_pos=torch.zeros(6, dtype=torch.int32, device=DEV))
    out_index = i32([0, 4, 2, 9, 1])
    temps = torch.tensor([0.0, 0.9, 0.0, 1.3, 0.0], device=DEV)
    seeds = torch.tensor([5, 6, 7, 8, 9], dtype=torch.int64, device=DEV)
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    advance = tuple(d[k] for k in ("token_ids", "positions", "seq_lens", "q_req", "slot_mapping", "block_tables",
                                   "page_sizes", "history", "history_pos"))
    want_tokens = []
    for step in range(2):
        logits = rnd(g, rows, vocab, scale=2.0)
        idx_before = out_index.cpu().tolist()
        kernels.sample(logits.to(DEV), rows, vocab, temps, None, None, seeds, out_index, 3, out, advance=advance)
        plain = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
        kernels.sample(logits.to(DEV), rows, vocab, temps, None, None, seeds, i32(idx_before), 3, plain)
        assert torch.equal(out, plain), "advancing must not change what is sampled"
        want_tokens.append(plain.cpu().tolist())
        for r in range(rows):
            if q_req[r] < 0:
                assert d["token_ids"][r].item() == tok0[r].item() and d["positions"][r].item() == positions[r]
                assert d["history_pos"][r].item() == 0 and out_index[r].item() == 2
                assert d["slot_mapping"][:, r].cpu().tolist() == [-7, -7]
                continue
            pos = positions[r] + step + 1
            assert d["token_ids"][r].item() == want_tokens[step][r]
            assert d["positions"][r].item() == pos and d["seq_lens"][r].item() == pos + 1
            assert out_index[r].item() == idx_before[r] + 1
            assert d["history_pos"][r].item() == step + 1 and d["history"][step, r].item() == want_tokens[step][r]
            for grp, ps in enumerate(page_sizes):
                page = bt[grp, r, pos // ps].item() if pos // ps < max_blocks else -1
                assert d["slot_mapping"][grp, r].item() == (page * ps + pos % ps if page >= 0 else -1)
    assert (d["history"][2] == -5).all() and (d["history"][:, 5] == -5).all()


@pytest.mark.parametrize("vocab", [257, 503, 5000])
def test_seeded_sampling_matches_the_plain_sampler(vocab):
    g = torch.Generator().manual_seed(9)
    m = 24
    logits = rnd(g, m, vocab, scale=2.0)
    temps = [0.8, 1.0, 0.3, 1.7] * (m // 4)
    top_k = [0, 5, 0, 40, 1, 0] * (m // 6)
    top_p = [1.0, 1.0, 0.7, 0.9, 1.0, 0.2] * (m // 6)
    seeds, idx = list(range(100, 100 + m)), [3 * i for i in range(m)]
    got = _sample(logits, temps, top_k, top_p, seeds, idx, engine_seed=42)
    assert got == _sample(logits, temps, top_k, top_p, seeds, idx, engine_seed=42)       # deterministic
    for r in range(m):
        u = P.plain_uniform(42, seeds[r], idx[r])
        tok, lo, hi, total = P.plain_sample(logits[r].numpy(), temps[r], top_k[r] or None,
                                            top_p[r] if top_p[r] < 1 else None, u)
        if got[r] != tok:
            # float32 prefix sums may move a boundary by rounding: then u must sit on that boundary
            edge = min(abs(u * total - lo), abs(u * total - hi))
            assert edge <= 1e-4 * total, f"row {r}: kernel {got[r]}, plain {tok}, u {u}"


def test_reference_vectors_top_k_top_p():
    # reference tests/test_sampling.py:25-38
    logits = torch.tensor([[1.0, 5.0, 3.0, 2.0, 4.0]] * 64)
    got = set(_sample(logits, [1.0] * 64, top_k=[2] * 64, seeds=list(range(64)), idx=[0] * 64))
    assert got == {1, 4}
    logits = torch.tensor([[10.0, 0.0, 0.0, 0.0]] * 64)
    assert set(_sample(logits, [1.0] * 64, top_p=[1e-6] * 64, seeds=list(range(64)), idx=[0] * 64)) == {0}
    # mixed rows: greedy beside stochastic (reference test_sampling.py:56-63)
    g = torch.Generator().manual_seed(10)
    logits = rnd(g, 2, 30)
    assert _sample(logits, [0.0, 1.0], seeds=[1, 2], idx=[0, 0])[0] == int(torch.argmax(logits[0]))


def test_sampling_follows_the_distribution():
    probs = torch.tensor([0.5, 0.25, 0.125, 0.125])
    m = 4096
    logits = probs.log().repeat(m, 1)
    got = np.bincount(_sample(logits, [1.0] * m, seeds=[7] * m, idx=list(range(m))), minlength=4) / m
    assert np.abs(got - probs.numpy()).max() < 0.03
