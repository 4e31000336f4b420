"""The entry point that allocates nothing (mgpt_linear_skinny_static_scratch) against the one it is a
variant of (mgpt_linear_skinny with the caller's scratch), called through ctypes: two calls in a
row, the second with a smaller input, and a shape beyond the library's array."""

import ctypes

import pytest
import torch

from mini_gpt_inference_amd.ops import kernels, library

pytestmark = pytest.mark.gpu

SHARE_W = kernels.ROWS_SHARE_W
ERR_SCRATCH = -5


def _both(n_rows, n_out, k_dim, epilogue, seed):
    """Runs the product through both entry points; returns (existing, static-scratch) outputs."""
    lib = library.kernels()
    fn = lib.mgpt_linear_skinny_static_scratch
    P, I, L, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
    fn.argtypes = [P, L, P, P, P, F, P, P, P, P, I, L, I, I, I, I, P, P, P, I, I, I, I, I, I, P]
    fn.restype = I
    g = torch.Generator(device="cuda").manual_seed(seed)
    act = (torch.randn(n_rows, k_dim, device="cuda", generator=g) * 0.5).to(torch.bfloat16)
    w = (torch.randn(n_out, k_dim, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    bias = torch.randn(n_out, device="cuda", generator=g)
    res = torch.randn(n_rows, n_out, device="cuda", generator=g)
    need = kernels.linear_skinny_partials(n_rows, n_out, k_dim, False, epilogue)
    if need == 0:      # left to itself the library deals these rows out in groups; ask for shared W
        need = 4 * n_rows * n_out
    outs = []
    for static in (False, True):
        out = res.clone() if epilogue == kernels.EPI_RESIDUAL else torch.zeros(n_rows, n_out, device="cuda",
                                                                              dtype=torch.bfloat16)
        if static:
            torch.cuda.synchronize()
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            rc = fn(act.data_ptr(), act.stride(0), None, None, None, 0.0, w.data_ptr(), None, bias.data_ptr(),
                    out.data_ptr(), kernels.F32 if out.dtype == torch.float32 else kernels.BF16, out.stride(0),
                    n_rows, n_out, k_dim, epilogue, None, None, None, 0, 0, 0, 0, 0, SHARE_W, stream)
            assert rc == 0, rc
        else:
            partials = torch.full((need,), float("nan"), device="cuda")
            assert kernels.linear_skinny(act, w, bias, out, n_rows, epilogue, partials=partials, rows_mode=SHARE_W)
        torch.cuda.synchronize()
        outs.append(out.float())
    ref = act.double() @ w.double().T + bias.double()
    if epilogue == kernels.EPI_RESIDUAL:
        ref = ref + res.double()
    if epilogue == kernels.EPI_GELU:
        ref = torch.nn.functional.gelu(ref, approximate="tanh")
    assert (outs[0].double() - ref).abs().max() <= 2e-2 * max(1.0, ref.abs().max().item())
    return outs


def test_static_scratch_entry_point_equals_the_callers_scratch_on_two_calls_in_a_row():
    lib = library.kernels()
    lib.mgpt_linear_skinny_static_scratch_floats.restype = ctypes.c_long
    assert lib.mgpt_linear_skinny_static_scratch_floats() == 4 * 64 * 1024
    # the array keeps what the first call left in it: the second, smaller call must not read any of that
    first = _both(64, 512, 2048, kernels.EPI_RESIDUAL, seed=1)
    assert torch.equal(first[0], first[1])
    second = _both(40, 256, 1024, kernels.EPI_GELU, seed=2)
    assert torch.equal(second[0], second[1])
    again = _both(64, 512, 2048, kernels.EPI_RESIDUAL, seed=1)
    assert torch.equal(again[1], first[1])


def test_static_scratch_entry_point_refuses_what_its_array_cannot_hold():
    lib = library.kernels()
    fn = lib.mgpt_linear_skinny_static_scratch
    P, I, L, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
    fn.argtypes = [P, L, P, P, P, F, P, P, P, P, I, L, I, I, I, I, P, P, P, I, I, I, I, I, I, P]
    fn.restype = I
    n_rows, n_out, k_dim = 64, 1536, 2048      # 4 * 64 * 1536 floats of partial sums
    act = torch.zeros(n_rows, k_dim, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(n_out, k_dim, device="cuda", dtype=torch.bfloat16)
    out = torch.full((n_rows, n_out), 7.0, device="cuda")
    rc = fn(act.data_ptr(), act.stride(0), None, None, None, 0.0, w.data_ptr(), None, None, out.data_ptr(),
            kernels.F32, out.stride(0), n_rows, n_out, k_dim, kernels.EPI_NONE, None, None, None, 0, 0, 0, 0, 0,
            SHARE_W, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == ERR_SCRATCH
    torch.cuda.synchronize()
    assert bool((out == 7.0).all()), "a refused call launches nothing"


def test_static_scratch_at_few_rows_under_a_long_inner_size_and_inside_a_captured_graph():
    """The split also comes at 16 rows or fewer under a long inner size with few column tiles, and
    the entry point is meant for code under graph capture: after the init call (which asks the
    runtime for the array's address outside any capture) a call captured into a graph gives the
    eager result on every replay, with other work on the array between the replays."""
    lib = library.kernels()
    lib.mgpt_linear_skinny_static_scratch_init.restype = ctypes.c_int
    assert lib.mgpt_linear_skinny_static_scratch_init() == 0
    n_rows, n_out, k_dim = 8, 1600, 6400
    assert kernels.linear_skinny_partials(n_rows, n_out, k_dim, False, kernels.EPI_RESIDUAL) > 0
    few = _both(n_rows, n_out, k_dim, kernels.EPI_RESIDUAL, seed=3)
    assert torch.equal(few[0], few[1])
    fn = lib.mgpt_linear_skinny_static_scratch
    g = torch.Generator(device="cuda").manual_seed(4)
    act = (torch.randn(n_rows, k_dim, device="cuda", generator=g) * 0.5).to(torch.bfloat16)
    w = (torch.randn(n_out, k_dim, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    out = torch.zeros(n_rows, n_out, device="cuda", dtype=torch.bfloat16)

    def call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = fn(act.data_ptr(), act.stride(0), None, None, None, 0.0, w.data_ptr(), None, None, out.data_ptr(),
                kernels.BF16, out.stride(0), n_rows, n_out, k_dim, kernels.EPI_NONE, None, None, None, 0, 0, 0, 0, 0,
                SHARE_W, stream)
        assert rc == 0, rc

    call()
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        graph.capture_begin()
        call()
        graph.capture_end()
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        out.fill_(7.0)
        _both(64, 512, 2048, kernels.EPI_RESIDUAL, seed=5)      # eager work that leaves other sums in the array
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
