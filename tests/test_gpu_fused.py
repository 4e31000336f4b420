"""The fused kernels of a decode step with few rows, each alone against the plain functions, at sizes
other than the engine's: a residual that arrives as a base plus pending partial sums (or as table
rows), widths, head sizes and counts that are no powers of two, contexts around the edges of a
wave's share of keys and of a pass, a far key that decides the softmax, NaN in everything a kernel
must not read, padded tokens."""

import math

import pytest
import torch

import helpers
import plain_gpt as P
from mini_gpt_inference_amd.ops import kernels
from mini_gpt_inference_amd.ops.residual import PendingSums

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rnd(gen, *shape, scale=1.0):
    return torch.randn(*shape, generator=gen, dtype=torch.float32) * scale


def bf(t):
    return t.to(torch.bfloat16)


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def _pending(gen, rows, width, n_parts, extra_rows=2):
    """A residual as the kernels before would have left it: base + parts, with rows of padding behind
    that hold NaN.  Returns (PendingSums on the device, the rows' true values in float64)."""
    base = rnd(gen, rows + extra_rows, width, scale=2.0) + 0.5
    base[rows:] = float("nan")
    parts = rnd(gen, max(n_parts, 1), rows + extra_rows, width, scale=0.7)
    parts[:, rows:] = float("nan")
    true = base[:rows].double() + (parts[:n_parts, :rows].double().sum(0) if n_parts else 0)
    return PendingSums(base.to(DEV), parts.to(DEV) if n_parts else None, n_parts), true


ATTN_CASES = [
    # width, heads, head size, page, contexts (keys before the token's own), parts of the residual, biases
    dict(c=512, h=8, d=64, page=16, ctx=[256, 0, 1, 31, 32, 33, 511, 512, 513, 700], parts=8, bias=True),
    dict(c=512, h=8, d=64, page=16, ctx=[5, 130], parts=32, bias=True),
    dict(c=96, h=3, d=32, page=8, ctx=[0, 17, 100, 515], parts=3, bias=False),
    dict(c=64, h=4, d=16, page=4, ctx=[60, 3, 1029], parts=4, bias=True),
    dict(c=256, h=2, d=128, page=32, ctx=[40, 600], parts=0, bias=True),
    dict(c=320, h=5, d=64, page=16, ctx=[77, 0, 300], parts=12, bias=False),
    dict(c=128, h=6, d=32, page=2, ctx=[9, 64], parts=1, bias=True),     # heads * head size wider than the model
    # more (token, head) pairs than compute units: two tokens a workgroup (more than 256 pairs) or four
    # (more than 512; heads of 128 keep to two); workgroups of real tokens and padded ones, and of
    # padded tokens only
    dict(c=512, h=8, d=64, page=16, ctx=[(7 * i * i + 3 * i) % 600 for i in range(45)], parts=8, bias=True, pad=3),
    dict(c=96, h=3, d=32, page=8, ctx=[(5 * i * i + i) % 300 for i in range(90)], parts=3, bias=False, pad=1),
    dict(c=64, h=4, d=16, page=4, ctx=[(11 * i * i) % 1100 for i in range(70)], parts=4, bias=True, pad=2),
    dict(c=256, h=2, d=128, page=32, ctx=[(3 * i * i + 2) % 400 for i in range(131)], parts=0, bias=True, pad=1),
    dict(c=512, h=8, d=64, page=16, ctx=[(7 * i * i + 3 * i) % 530 for i in range(65)], parts=32, bias=True, pad=6),
    dict(c=64, h=4, d=16, page=4, ctx=[(13 * i * i) % 270 for i in range(141)], parts=4, bias=False, pad=1),
    dict(c=96, h=3, d=32, page=8, ctx=[(5 * i * i + 7 * i) % 200 for i in range(175)], parts=2, bias=True, pad=3),
    dict(c=256, h=2, d=128, page=32, ctx=[(3 * i) % 40 for i in range(253)], parts=1, bias=True, pad=1),
]


@pytest.mark.parametrize("tables", [False, True])
@pytest.mark.parametrize("case", range(len(ATTN_CASES)))
def test_fused_attention_decode(case, tables):
    spec = ATTN_CASES[case]
    c, h, d, page, ctxs = spec["c"], spec["h"], spec["d"], spec["page"], spec["ctx"]
    g = torch.Generator().manual_seed(100 + case)
    n = len(ctxs)
    pad = spec.get("pad", 1)
    rows = n + pad                                # padded tokens behind the real ones
    qw = h * d
    gain, beta = 1 + 0.1 * rnd(g, c), rnd(g, c, scale=0.1)
    wqkv, wproj = bf(rnd(g, 3 * qw, c, scale=c ** -0.5)), bf(rnd(g, c, qw, scale=qw ** -0.5))
    bqkv, bproj = (rnd(g, 3 * qw, scale=0.2), rnd(g, c, scale=0.2)) if spec["bias"] else (None, None)
    eps, scale = 1e-5, (0.21 if case % 2 else 1.0 / math.sqrt(d))
    if tables:
        vocab, n_pos = 61, max(ctxs) + 1
        tok, pos = bf(rnd(g, vocab, c)), bf(rnd(g, n_pos, c, scale=0.5))
        ids = torch.randint(0, vocab, (rows,), generator=g)
        pending = PendingSums(None, None, 0, (tok.to(DEV), pos.to(DEV), i32(ids), i32(ctxs + [0] * pad)))
        true = tok.double()[ids[:n]] + pos.double()[ctxs]
    else:
        pending, true = _pending(g, n, c, spec["parts"], extra_rows=pad)
    # many (token, head) pairs: a workgroup takes several tokens, and rows that are no table rows come normed
    several = kernels.fused_attention_tokens(rows, h, d) > 1
    assert several == (rows * h > 256)
    normed = None
    if several and not tables:
        assert not kernels.fused_attention_decode(          # the pending parts are refused, nothing is launched
            pending, torch.zeros(rows, c, device=DEV), gain.to(DEV), beta.to(DEV), eps,
            torch.zeros(3 * qw * c, dtype=torch.bfloat16, device=DEV), None,
            torch.zeros(c * qw, dtype=torch.bfloat16, device=DEV), None, torch.zeros(h, rows, c, device=DEV),
            torch.zeros(4, h, page, d, dtype=torch.bfloat16, device=DEV),
            torch.zeros(4, h, page, d, dtype=torch.bfloat16, device=DEV), i32([-1] * rows),
            torch.zeros(rows, 4, dtype=torch.int32, device=DEV), i32([0] * rows), i32([-1] * rows), rows, h, scale)
        plain_rows = torch.full((rows, c), float("nan"))
        plain_rows[:n] = true.float()
        true = plain_rows[:n].double()
        pending = PendingSums(plain_rows.to(DEV), None, 0)
        normed = torch.full((rows, c), float("nan"), dtype=torch.bfloat16)
        normed[:n] = bf(P.plain_layer_norm(true, gain.double(), beta.double(), eps))
        normed = normed.to(DEV)
    # the cache: every request's earlier keys and values in pages handed out in a shuffled order
    max_blocks = max(-(-(x + 1) // page) for x in ctxs) + 1
    n_pages = sum(-(-(x + 1) // page) for x in ctxs) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    kp = torch.full((n_pages, h, page, d), float("nan"), dtype=torch.bfloat16)
    vp = kp.clone()
    bt = torch.full((rows, max_blocks), 10 ** 6, dtype=torch.int32)      # unused entries point far outside the pool
    past_k, past_v, slots = [], [], []
    for r, ctx in enumerate(ctxs):
        k_r, v_r = bf(rnd(g, ctx, h, d)), bf(rnd(g, ctx, h, d))
        past_k.append(k_r)
        past_v.append(v_r)
        for b in range(-(-(ctx + 1) // page)):
            bt[r, b] = order.pop()
        for t in range(ctx):
            kp[bt[r, t // page], :, t % page] = k_r[t]
            vp[bt[r, t // page], :, t % page] = v_r[t]
        slots.append(int(bt[r, ctx // page]) * page + ctx % page)
    # what the kernel must compute, in float64 from the rounded inputs
    hn = P.plain_layer_norm(true, gain.double(), beta.double(), eps)
    qkv = P.plain_linear(bf(hn).double(), wqkv.double(), None if bqkv is None else bqkv.double())
    # a far key decides the first long request's softmax: a key at position 3 that points along the query
    far = next((r for r, ctx in enumerate(ctxs) if ctx > 200), None)
    if far is not None:
        qf = bf(qkv[far, :d]).double()
        key = bf((6.0 / scale / qf.norm() ** 2 * qf).float())
        past_k[far][3, 0] = key
        kp[bt[far, 3 // page], 0, 3 % page] = key
    want = torch.empty(n, c, dtype=torch.float64)
    for r, ctx in enumerate(ctxs):
        q, k, v = P.plain_split_heads(bf(qkv[r:r + 1]).double(), h)
        keys = torch.cat([past_k[r].double().transpose(0, 1), k], dim=1)        # [H, ctx + 1, D]
        vals = torch.cat([past_v[r].double().transpose(0, 1), v], dim=1)
        y = P.plain_causal_attention(q, keys, vals, scale=scale, causal=False)   # one query sees all ctx + 1 keys
        want[r] = P.plain_linear(bf(y).double(), wproj.double(), None if bproj is None else bproj.double())
    dev = lambda t: None if t is None else t.to(DEV)
    settled = torch.full((rows, c), float("nan"), device=DEV)
    out = torch.full((h, rows, c), float("nan"), device=DEV)
    kp_d, vp_d = kp.to(DEV), vp.to(DEV)
    took = kernels.fused_attention_decode(
        pending, settled, dev(gain), dev(beta), eps, kernels.pack_weight(wqkv.to(DEV)), dev(bqkv),
        kernels.pack_weight(wproj.to(DEV)), dev(bproj), out, kp_d, vp_d, i32(slots + [-1] * pad), bt.to(DEV),
        i32(ctxs + [0] * pad), i32(list(range(n)) + [-1] * pad), rows, h, scale, normed=normed)
    assert took
    torch.cuda.synchronize()
    if normed is None:
        helpers.assert_close(settled[:n], true, "float32", "the settled rows")
    else:
        assert torch.isnan(settled).all(), "rows that came normed are not stored again"
    helpers.assert_close(out[:, :n].sum(0), want, "bfloat16", f"fused attention case {case}")
    assert torch.isnan(out[:, n:]).all() and torch.isnan(settled[n:]).all(), "the padded tokens' rows were written"
    for r, ctx in enumerate(ctxs):                 # the token's key and value are in its page, nothing else changed
        page_i, off = slots[r] // page, slots[r] % page
        _, k, v = P.plain_split_heads(qkv[r:r + 1], h)
        helpers.assert_close(kp_d[page_i, :, off], k[:, 0], "bfloat16", "the stored key")
        helpers.assert_close(vp_d[page_i, :, off], v[:, 0], "bfloat16", "the stored value")
        kp[page_i, :, off] = kp_d[page_i, :, off].cpu()
        vp[page_i, :, off] = vp_d[page_i, :, off].cpu()
    same = lambda a, b: torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert same(kp_d.cpu(), kp) and same(vp_d.cpu(), vp), "the cache changed beyond the new slots"


MLP_CASES = [
    # width, hidden, rows, parts of the residual, biases
    dict(c=512, f=2048, rows=1, parts=8, bias=True),
    dict(c=512, f=2048, rows=8, parts=8, bias=True),
    dict(c=512, f=2048, rows=16, parts=8, bias=False),
    dict(c=512, f=2048, rows=23, parts=12, bias=True),      # more parts than a wave adds: fewer rows a workgroup
    dict(c=96, f=384, rows=5, parts=3, bias=False),
    dict(c=64, f=256, rows=3, parts=0, bias=True),
    dict(c=320, f=1280, rows=9, parts=5, bias=True),
    dict(c=256, f=64, rows=2, parts=40, bias=True),
    dict(c=128, f=8192, rows=40, parts=2, bias=True),       # more workgroups than compute units
]


@pytest.mark.parametrize("case", range(len(MLP_CASES)))
def test_fused_mlp_decode(case):
    spec = MLP_CASES[case]
    c, f, rows = spec["c"], spec["f"], spec["rows"]
    g = torch.Generator().manual_seed(200 + case)
    pending, true = _pending(g, rows, c, spec["parts"])
    gain, beta = 1 + 0.1 * rnd(g, c), rnd(g, c, scale=0.1)
    wfc, wproj = bf(rnd(g, f, c, scale=c ** -0.5)), bf(rnd(g, c, f, scale=f ** -0.5))
    bfc, bproj = (rnd(g, f, scale=0.3), rnd(g, c, scale=0.3)) if spec["bias"] else (None, None)
    eps = 1e-6 if case % 2 else 1e-5
    hn = bf(P.plain_layer_norm(true, gain.double(), beta.double(), eps)).double()
    u = P.plain_gelu_tanh(P.plain_linear(hn, wfc.double(), None if bfc is None else bfc.double()))
    want = P.plain_linear(bf(u).double(), wproj.double(), None if bproj is None else bproj.double())
    dev = lambda t: None if t is None else t.to(DEV)
    n_parts = kernels.fused_mlp_parts(f)
    assert n_parts == f // 64
    settled = torch.full((rows + 2, c), float("nan"), device=DEV)
    out = torch.full((n_parts, rows + 2, c), float("nan"), device=DEV)
    took = kernels.fused_mlp_decode(pending, settled, dev(gain), dev(beta), eps, kernels.pack_weight(wfc.to(DEV)),
                                    dev(bfc), kernels.pack_weight(wproj.to(DEV)), dev(bproj), out, rows, f)
    assert took
    torch.cuda.synchronize()
    helpers.assert_close(settled[:rows], true, "float32", "the settled rows")
    helpers.assert_close(out[:, :rows].sum(0), want, "bfloat16", f"fused feed-forward case {case}")
    assert torch.isnan(out[:, rows:]).all() and torch.isnan(settled[rows:]).all(), "rows beyond the step were written"


@pytest.mark.parametrize("out_dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("c,parts,bias", [(512, 32, True), (96, 3, False), (64, 0, True), (320, 12, True), (32, 100, True),
                                          (768, 20, True), (1600, 4, True), (1600, 8, False), (4096, 4, True), (2080, 0, True)])
def test_residual_layer_norm_and_settle(c, parts, bias, out_dtype):
    g = torch.Generator().manual_seed(300 + c)
    rows = 7
    pending, true = _pending(g, rows, c, parts)
    gain, beta = 1 + 0.1 * rnd(g, c), rnd(g, c, scale=0.1) if bias else None
    want = P.plain_layer_norm(true, gain.double(), None if beta is None else beta.double(), 1e-5)
    dev = lambda t: None if t is None else t.to(DEV)
    tdt = torch.float32 if out_dtype == "float32" else torch.bfloat16
    out = torch.full((rows, c), float("nan"), dtype=tdt, device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, None, out, rows)
    helpers.assert_close(out, want, out_dtype, "LayerNorm of a pending residual")
    pick = [6, 0, 3, 3]
    out2 = torch.full((4, c), float("nan"), dtype=tdt, device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, i32(pick), out2, 4)
    helpers.assert_close(out2, want[pick], out_dtype, "LayerNorm of chosen rows of a pending residual")
    # the LayerNorm that goes over all rows can store the sums on its way: into another array ...
    out3 = torch.full((rows, c), float("nan"), dtype=tdt, device=DEV)
    stored = torch.full((rows + 2, c), float("nan"), device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, None, out3, rows, settled=stored)
    assert torch.equal(out3, out)
    helpers.assert_close(stored[:rows], true, "float32", "sums stored by the LayerNorm")
    assert torch.isnan(stored[rows:]).all()
    # the sum itself: into another array, and into the base
    settled = torch.full((rows + 2, c), float("nan"), device=DEV)
    assert kernels.residual_settle(pending, settled, rows)
    helpers.assert_close(settled[:rows], true, "float32", "settle")
    assert torch.isnan(settled[rows:]).all()
    # ... and into the base itself (a workgroup is the only reader of its row)
    keep = pending.base.clone()
    out4 = torch.full((rows, c), float("nan"), dtype=tdt, device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, None, out4, rows, settled=pending.base)
    assert torch.equal(out4, out) and torch.equal(pending.base[:rows], stored[:rows])
    pending.base.copy_(keep)
    assert kernels.residual_settle(pending, pending.base, rows)
    helpers.assert_close(pending.base[:rows], true, "float32", "settle in place")


def test_residual_kernels_say_which_widths_and_parts_they_take():
    assert kernels.residual_parts_limit(512) == 32 and kernels.residual_parts_limit(1600) == 8
    assert kernels.residual_parts_limit(4096) == 4 and kernels.residual_parts_limit(4128) == 0
    assert kernels.residual_parts_limit(1616) == 0          # no multiple of 32
    g = torch.Generator().manual_seed(9)
    for c, parts in ((1600, 9), (4128, 1), (1616, 1)):
        base = rnd(g, 2, c).to(DEV)
        pending = PendingSums(base, rnd(g, parts, 2, c).to(DEV), parts)
        out = torch.full((2, c), 7.0, device=DEV)
        assert not kernels.residual_layer_norm(pending, torch.ones(c, device=DEV), None, 1e-5, None, out, 2)
        assert (out == 7.0).all()


@pytest.mark.parametrize("rows,n_out,k_dim,bias,packed", [(1, 1600, 6400, True, True), (8, 768, 3072, True, True),
                                                        (16, 512, 4096, False, False), (40, 1600, 6400, True, True),
                                                        (5, 96, 3072, True, False)])
def test_split_product_left_as_parts_of_a_pending_residual(rows, n_out, k_dim, bias, packed):
    """The split product's first kernel alone: its parts (the first carries the bias) add up to the
    plain product, in the order of k to the very bits that the two-kernel product stores; and the
    residual LayerNorm that reads base + parts gives the LayerNorm of x + product."""
    g = torch.Generator().manual_seed(rows + n_out)
    a = bf(rnd(g, rows, k_dim))
    w = bf(rnd(g, n_out, k_dim, scale=0.03))
    b = rnd(g, n_out) if bias else None
    x = rnd(g, rows + 1, n_out, scale=2.0)
    x[rows:] = float("nan")
    dev = lambda t: None if t is None else t.to(DEV)
    wd = dev(w)
    need = kernels.linear_skinny_partials(rows, n_out, k_dim, False, kernels.EPI_RESIDUAL)
    assert need == 4 * rows * n_out
    parts = torch.full((4, rows, n_out), float("nan"), device=DEV)
    wp = kernels.pack_weight(wd) if packed else None
    assert kernels.linear_decode_parts(dev(a), wd, dev(b), parts, rows, w_packed=wp) == 4
    want = P.plain_linear(a.double(), w.double(), None if b is None else b.double())
    helpers.assert_close(parts.sum(0), want, "bfloat16", "sum of the parts")
    # the same sums as the product that adds them up itself (parts in the order of k, then the bias)
    two = torch.zeros(rows, n_out, device=DEV)
    scratch = torch.zeros(need, device=DEV)
    assert kernels.linear_skinny(dev(a), wd, dev(b), two, rows, kernels.EPI_NONE, partials=scratch, w_packed=wp)
    raw = scratch.view(4, rows, n_out)
    assert torch.equal(parts[1:], raw[1:])
    if b is None:
        assert torch.equal(parts[0], raw[0])
    else:
        assert torch.equal(parts[0], raw[0] + dev(b))
    # read as a pending residual
    pending = PendingSums(dev(x), parts, 4)
    gain, beta = 1 + 0.1 * rnd(g, n_out), rnd(g, n_out, scale=0.1)
    out = torch.full((rows, n_out), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, None, out, rows, settled=pending.base)
    true = x[:rows].double() + want
    helpers.assert_close(pending.base[:rows], true, "bfloat16", "x + product")
    assert torch.isnan(pending.base[rows:]).all()
    helpers.assert_close(out, P.plain_layer_norm(pending.base[:rows].double().cpu(), gain.double(), beta.double(), 1e-5),
                         "bfloat16", "LayerNorm of x + product")


@pytest.mark.parametrize("rows,n_out,k_dim,bias", [(48, 1600, 6400, True), (64, 1600, 6400, False), (33, 768, 3072, True),
                                                   (100, 512, 4096, True), (129, 1600, 6400, True),
                                                   (200, 1600, 6400, False), (256, 1600, 6400, True),
                                                   (160, 768, 3072, True), (256, 768, 3072, False)])
def test_tiled_split_left_as_parts_of_a_pending_residual(rows, n_out, k_dim, bias):
    """The tiled product's first kernel alone where it splits the inner size: its parts (the first
    carries the bias) add up to the plain product, to the very bits of the product that joins them
    itself; the residual LayerNorm that reads base + parts gives the LayerNorm of x + product."""
    g = torch.Generator().manual_seed(rows + n_out)
    a = bf(rnd(g, rows, k_dim))
    w = bf(rnd(g, n_out, k_dim, scale=0.03))
    b = rnd(g, n_out) if bias else None
    x = rnd(g, rows + 1, n_out, scale=2.0)
    x[rows:] = float("nan")
    dev = lambda t: None if t is None else t.to(DEV)
    wd = dev(w)
    need = kernels.linear_mfma_partials(rows, n_out, k_dim, kernels.EPI_RESIDUAL)
    n_parts = need // (rows * n_out)
    assert n_parts > 1 and need == n_parts * rows * n_out
    parts = torch.full((n_parts, rows, n_out), float("nan"), device=DEV)
    assert kernels.linear_mfma_parts(dev(a), wd, dev(b), parts, rows)
    want = P.plain_linear(a.double(), w.double(), None if b is None else b.double())
    helpers.assert_close(parts.sum(0), want, "bfloat16", "sum of the parts")
    joined = torch.zeros(rows, n_out, device=DEV)
    scratch = torch.zeros(need, device=DEV)
    # (from 128 rows on the library, left to itself, does not split such a product: it sends the slices
    # straight into LDS, four steps deep; the split is asked for then)
    assert kernels.linear_mfma(dev(a), wd, dev(b), joined, rows, kernels.EPI_NONE, partials=scratch,
                               k_parts=None if rows < 128 else n_parts)
    raw = scratch.view(n_parts, rows, n_out)
    if rows < 128:
        assert torch.equal(parts[1:], raw[1:])
    else:   # (the split that is asked for may take other tiles, whose waves add a step's halves in another order)
        helpers.assert_close(parts[1:], raw[1:], "float32", "the parts of the split that was asked for")
    helpers.assert_close(parts[0], raw[0].double().cpu() + (0 if b is None else b.double()), "float32", "the first part")
    # read as a pending residual
    pending = PendingSums(dev(x), parts, n_parts)
    gain, beta = 1 + 0.1 * rnd(g, n_out), rnd(g, n_out, scale=0.1)
    out = torch.full((rows, n_out), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert kernels.residual_layer_norm(pending, dev(gain), dev(beta), 1e-5, None, out, rows, settled=pending.base)
    true = x[:rows].double() + want
    helpers.assert_close(pending.base[:rows], true, "bfloat16", "x + product")
    assert torch.isnan(pending.base[rows:]).all()
    helpers.assert_close(out, P.plain_layer_norm(pending.base[:rows].double().cpu(), gain.double(), beta.double(), 1e-5),
                         "bfloat16", "LayerNorm of x + product")
    # a product that the tiled kernel does not split leaves no parts
    small = torch.full((2, rows, 4096), 7.0, device=DEV)
    assert not kernels.linear_mfma_parts(dev(a)[:, :512].contiguous(), bf(rnd(g, 4096, 512)).to(DEV), None, small, rows)
    assert bool((small == 7.0).all())


def test_split_parts_are_refused_where_the_product_is_not_split():
    g = torch.Generator().manual_seed(2)
    for rows, n_out, k_dim in ((4, 512, 2048), (4, 4096, 4096), (70, 512, 4096)):
        a, w = bf(rnd(g, rows, k_dim)).to(DEV), bf(rnd(g, n_out, k_dim)).to(DEV)
        parts = torch.full((4, rows, n_out), 7.0, device=DEV)
        assert kernels.linear_decode_parts(a, w, None, parts, rows) == 0
        assert (parts == 7.0).all()


def test_fused_kernels_refuse_what_they_cannot_do():
    """Widths beyond 512 or no multiple of 32, more pending sums than a reader adds up on its way in,
    key/value groups, head sizes outside 16/32/64/128, a hidden size that is no multiple of 64: False,
    and nothing is written."""
    assert kernels.fused_parts_limit(512) == 32 and kernels.fused_parts_limit(544) == 0
    assert kernels.fused_parts_limit(48) == 0 and kernels.fused_parts_limit(64) >= 128
    # rows: up to four tokens a workgroup (two with heads of 128) and 256 workgroups a head's share
    assert [kernels.fused_attention_tokens(r, 8, 64) for r in (1, 32, 33, 64, 65, 128, 129)] == [1, 1, 2, 2, 4, 4, 0]
    assert [kernels.fused_attention_tokens(r, 2, 128) for r in (128, 129, 256, 257)] == [1, 2, 2, 0]
    g = torch.Generator().manual_seed(5)
    for c, f, parts in [(544, 2176, 2), (48, 192, 2), (512, 2048, 33), (512, 2000, 2)]:
        base = rnd(g, 2, c).to(DEV)
        pending = PendingSums(base, rnd(g, parts, 2, c).to(DEV), parts)
        out = torch.full((max(f // 64, 1), 2, c), 7.0, device=DEV)
        settled = torch.full((2, c), 7.0, device=DEV)
        w = torch.zeros(f * c, dtype=torch.bfloat16, device=DEV)
        assert not kernels.fused_mlp_decode(pending, settled, torch.ones(c, device=DEV), None, 1e-5, w, None, w, None,
                                            out, 2, f)
        torch.cuda.synchronize()
        assert bool((out == 7.0).all()) and bool((settled == 7.0).all())
        if c % 32 or parts > kernels.residual_parts_limit(c):      # (this kernel alone takes rows up to 4096 wide)
            assert not kernels.residual_layer_norm(pending, torch.ones(c, device=DEV), None, 1e-5, None,
                                                   torch.zeros(2, c, device=DEV), 2)
    # attention: two key/value heads under four query heads, and a head size of 48
    for hk, d in [(2, 64), (4, 48)]:
        c, h = 256, 4
        pending = PendingSums(rnd(g, 1, c).to(DEV), None, 0)
        pools = torch.zeros(4, hk, 16, d, dtype=torch.bfloat16, device=DEV)
        w1 = torch.zeros(3 * h * d * c, dtype=torch.bfloat16, device=DEV)
        w2 = torch.zeros(c * h * d, dtype=torch.bfloat16, device=DEV)
        out = torch.full((h, 1, c), 7.0, device=DEV)
        assert not kernels.fused_attention_decode(pending, torch.zeros(1, c, device=DEV), torch.ones(c, device=DEV), None,
                                                  1e-5, w1, None, w2, None, out, pools, pools.clone(), i32([0]),
                                                  torch.zeros(1, 4, dtype=torch.int32, device=DEV), i32([0]), i32([0]),
                                                  1, h, 0.125)
        assert bool((out == 7.0).all())
