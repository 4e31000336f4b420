"""Typed Python entry points of the HIP kernels.

Each function checks on the host that operand shapes, strides, dtypes and
devices are what the kernel and its grid assume, then launches on the current
HIP stream.  Tensors are torch tensors used as plain device buffers; no torch
operator computes anything here.
"""

from __future__ import annotations

import contextlib
import ctypes
from typing import Dict, Optional

import torch

from . import library

F32, BF16 = 0, 1
EPI_NONE, EPI_GELU, EPI_RESIDUAL = 0, 1, 2

_ERRORS = {
    -1: "unsupported dtype combination",
    -2: "unsupported shape",
    -3: "size beyond what the launch grid can hold",
    -4: "null pointer",
    -5: "the shape needs more scratch than the library's own array holds",
}


class KernelError(RuntimeError):
    pass


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16 buffers, got {t.dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    """The address for a pointer argument (ctypes takes an int, or None for null, where argtypes say c_void_p)."""
    return None if t is None else t.data_ptr()


_pinned_stream: Optional[ctypes.c_void_p] = None


def _stream() -> ctypes.c_void_p:
    if _pinned_stream is not None:
        return _pinned_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


@contextlib.contextmanager
def pinned_stream():
    """Inside the block every launch goes to the stream that is current on entry.  Asking torch for
    the current stream costs about as much as a launch does, and a step is some hundred launches;
    the block must not switch streams."""
    global _pinned_stream
    previous = _pinned_stream
    _pinned_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    try:
        yield
    finally:
        _pinned_stream = previous


launches = 0     # kernels launched so far (a product split over workgroups counts its second kernel too)


def _check(rc: int, what: str, n_kernels: int = 1) -> None:
    global launches
    if rc == 0:
        launches += n_kernels
        return
    if rc < 0:
        raise KernelError(f"{what}: refused, {_ERRORS.get(rc, rc)}")
    raise KernelError(f"{what}: HIP error {rc}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _need_cuda(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _need_i32(name: str, t: torch.Tensor, n: int) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n,
          f"{name} must be a contiguous int32 buffer of at least {n} entries")


def embed(ids: torch.Tensor, positions: Optional[torch.Tensor], table: torch.Tensor,
          pos_table: Optional[torch.Tensor], x: torch.Tensor, n_tokens: int) -> None:
    """x[t] = table[ids[t]] (+ pos_table[positions[t]]), into the float32 residual stream."""
    _need_cuda(ids, positions, table, pos_table, x)
    width = table.shape[1]
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be dense [vocab, width]")
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] == width and x.shape[0] >= n_tokens,
          "residual stream must be dense float32 [>=n_tokens, width]")
    _need_i32("ids", ids, n_tokens)
    if pos_table is not None:
        _need(pos_table.dtype == table.dtype and pos_table.is_contiguous() and pos_table.shape[1] == width,
              "position table must match the token table's dtype and width")
        _need(positions is not None, "positions are needed with a position table")
        _need_i32("positions", positions, n_tokens)
    rc = library.kernels().mgpt_embed(_ptr(ids), _ptr(positions), _ptr(table), _ptr(pos_table), _ptr(x),
                                      n_tokens, width, _dtype_code(table), _stream())
    _check(rc, "embed")


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
               n_rows: int, eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """out[i] = LayerNorm(x[rows[i]] or x[i]); statistics in float32."""
    _need_cuda(x, weight, bias, out, rows)
    width = x.shape[1]
    _need(x.dtype == torch.float32 and x.is_contiguous(), "LayerNorm input must be dense float32")
    _need(weight.dtype == torch.float32 and weight.numel() == width, "LayerNorm weight must be float32 [width]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == width),
          "LayerNorm bias must be float32 [width]")
    _need(out.is_contiguous() and out.shape[1] == width and out.shape[0] >= n_rows, "LayerNorm output too small")
    if rows is None:
        _need(x.shape[0] >= n_rows, "LayerNorm input has fewer rows than asked for")
    else:
        _need_i32("rows", rows, n_rows)
    rc = library.kernels().mgpt_layernorm(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _ptr(rows), n_rows,
                                          width, float(eps), _dtype_code(out), _stream())
    _check(rc, "layer_norm")


def linear_generic(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                   n_rows: int, epilogue: int = EPI_NONE) -> None:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias), optional GELU, or added into a float32 out."""
    _need_cuda(a, w, bias, out)
    n_out, k_dim = w.shape
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          f"activation must be [>=n_rows, {k_dim}] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] == n_out and out.shape[0] >= n_rows,
          f"output must be [>=n_rows, {n_out}] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    rc = library.kernels().mgpt_linear_generic(
        _ptr(a), _dtype_code(a), a.stride(0), _ptr(w), _dtype_code(w), _ptr(bias), _ptr(out), _dtype_code(out),
        out.stride(0), n_rows, n_out, k_dim, epilogue, _stream())
    _check(rc, "linear_generic")


def kv_write(qkv: torch.Tensor, k_off: int, v_off: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
             slot_mapping: torch.Tensor, n_tokens: int) -> None:
    """Stores the new keys and values of n_tokens rows of qkv into their pages.

    Pools are [num_pages, n_kv_head, page_size, head_dim]."""
    _need_cuda(qkv, k_pool, v_pool, slot_mapping)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    _need(qkv.dtype == k_pool.dtype == v_pool.dtype, "pools must have the activations' dtype")
    _need(qkv.stride(1) == 1 and qkv.shape[0] >= n_tokens, "qkv rows must have unit inner stride")
    width = n_kv_head * head_dim
    _need(0 <= k_off and k_off + width <= qkv.shape[1] and 0 <= v_off and v_off + width <= qkv.shape[1],
          "key/value columns lie outside the qkv buffer")
    _need_i32("slot_mapping", slot_mapping, n_tokens)
    rc = library.kernels().mgpt_kv_write(_ptr(qkv), _dtype_code(qkv), qkv.stride(0), k_off, v_off, _ptr(k_pool),
                                         _ptr(v_pool), _ptr(slot_mapping), n_tokens, n_kv_head, head_dim,
                                         page_size, _stream())
    _check(rc, "kv_write")


def _check_attention_args(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head):
    _need_cuda(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    _need(q.dtype == out.dtype == k_pool.dtype == v_pool.dtype, "queries, output and pools must share a dtype")
    _need(q.stride(1) == 1 and out.stride(1) == 1, "query and output rows must have unit inner stride")
    _need(q.shape[0] >= n_tokens and out.shape[0] >= n_tokens, "query/output buffers have too few rows")
    _need(q.shape[1] >= n_head * head_dim and out.shape[1] >= n_head * head_dim,
          "query/output rows are narrower than n_head * head_dim")
    _need(n_head % n_kv_head == 0, "n_head must be a multiple of the number of key/value heads")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_req, "block_tables must be dense int32 [>=requests, max_blocks]")
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("seq_lens", seq_lens, n_req)
    _need_i32("q_req", q_req, n_tokens)
    return n_kv_head, page_size, head_dim


def paged_attention_generic(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor,
                            q_req: torch.Tensor, n_tokens: int, n_req: int, n_head: int, scale: float,
                            window: int = 0, fast_exp: bool = False) -> None:
    """Causal attention of the step's tokens over their requests' pages (any q_len, any dtype)."""
    n_kv_head, page_size, head_dim = _check_attention_args(
        q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head)
    _need(head_dim <= 256, f"head size {head_dim} exceeds the kernel's limit of 256")
    rc = library.kernels().mgpt_paged_attention_generic(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), _ptr(q_req), n_tokens, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), _dtype_code(q), int(fast_exp), _stream())
    _check(rc, "paged_attention_generic")


def sample(logits: torch.Tensor, n_rows: int, real_vocab: int, temperature: torch.Tensor,
           top_k: Optional[torch.Tensor], top_p: Optional[torch.Tensor], request_seed: Optional[torch.Tensor],
           out_index: Optional[torch.Tensor], engine_seed: int, out_tokens: torch.Tensor, advance=None,
           tile_best=None) -> None:
    """One token per row of float32 logits: argmax where temperature <= 0, else seeded sampling.

    tile_best = (values, columns), float32 and int32 [>=n_rows, tiles]: what linear_head_best left
    beside these logits with limit = real_vocab; greedy rows then read those instead of the logits.

    advance = (token_ids, positions, seq_lens, q_req, slot_mapping [groups, n_stride], block_tables
    [groups, r_stride, max_blocks], page_sizes [groups], history [rows, stride], history_pos): after
    a decode-only step each row also prepares the next step on the device (token, position, length,
    output index, cache slot) and appends its token to the history."""
    _need_cuda(logits, temperature, top_k, top_p, request_seed, out_index, out_tokens)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1 and logits.shape[0] >= n_rows,
          "logits must be float32 [>=n_rows, vocab] with unit inner stride")
    vocab = logits.shape[1]
    _need(0 < real_vocab <= vocab, "real_vocab must lie in 1..vocab")
    _need(temperature.dtype == torch.float32 and temperature.numel() >= n_rows, "temperature must be float32 [rows]")
    _need(top_k is None or (top_k.dtype == torch.int32 and top_k.numel() >= n_rows), "top_k must be int32 [rows]")
    _need(top_p is None or (top_p.dtype == torch.float32 and top_p.numel() >= n_rows), "top_p must be float32 [rows]")
    _need(request_seed is None or (request_seed.dtype in (torch.int64, torch.uint64) and request_seed.numel() >= n_rows),
          "request_seed must be 64-bit [rows]")
    _need(out_index is None or (out_index.dtype == torch.int32 and out_index.numel() >= n_rows),
          "out_index must be int32 [rows]")
    _need_i32("out_tokens", out_tokens, n_rows)
    tb = ti = None
    n_tiles = 0
    if tile_best is not None:
        tb, ti = tile_best
        _need_cuda(tb, ti)
        _need(tb.dtype == torch.float32 and ti.dtype == torch.int32 and tb.dim() == 2 and tb.is_contiguous()
              and ti.is_contiguous() and tb.shape == ti.shape and tb.shape[0] >= n_rows,
              "tile_best must be dense float32 values and int32 columns [>=n_rows, tiles]")
        n_tiles = tb.shape[1]
    if advance is not None:
        token_ids, positions, seq_lens, q_req, slot_mapping, block_tables, page_sizes, history, history_pos = advance
        _need_cuda(*advance)
        _need(out_index is not None, "advancing needs the output index array")
        _need(slot_mapping.dtype == torch.int32 and slot_mapping.dim() == 2 and slot_mapping.is_contiguous(),
              "slot_mapping must be dense int32 [groups, tokens]")
        n_groups, n_stride = slot_mapping.shape
        _need(block_tables.dtype == torch.int32 and block_tables.dim() == 3 and block_tables.is_contiguous()
              and block_tables.shape[0] == n_groups, "block_tables must be dense int32 [groups, requests, blocks]")
        _, r_stride, max_blocks = block_tables.shape
        _need(n_rows <= n_stride and n_rows <= r_stride, "more rows than the step's arrays hold")
        _need_i32("page_sizes", page_sizes, n_groups)
        _need(history.dtype == torch.int32 and history.dim() == 2 and history.is_contiguous()
              and history.shape[1] >= n_rows, "history must be dense int32 [steps, >=rows]")
        for name, t in (("token_ids", token_ids), ("positions", positions), ("seq_lens", seq_lens),
                        ("q_req", q_req), ("history_pos", history_pos)):
            _need_i32(name, t, n_rows)
        rc = library.kernels().mgpt_sample_advance(
            _ptr(logits), logits.stride(0), n_rows, vocab, real_vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
            _ptr(request_seed), _ptr(out_index), ctypes.c_ulonglong(engine_seed & (2**64 - 1)), _ptr(out_tokens),
            _ptr(token_ids), _ptr(positions), _ptr(seq_lens), _ptr(q_req), _ptr(slot_mapping), _ptr(block_tables),
            _ptr(page_sizes), n_groups, n_stride, r_stride, max_blocks, _ptr(history), _ptr(history_pos),
            history.shape[0], history.stride(0), _ptr(tb), _ptr(ti), n_tiles, _stream())
        _check(rc, "sample_advance")
        return
    rc = library.kernels().mgpt_sample(_ptr(logits), logits.stride(0), n_rows, vocab, real_vocab,
                                       _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(request_seed),
                                       _ptr(out_index), ctypes.c_ulonglong(engine_seed & (2**64 - 1)),
                                       _ptr(out_tokens), _ptr(tb), _ptr(ti), n_tiles, _stream())
    _check(rc, "sample")


SK_EPI_QKV = 3
_SKINNY_MAX_ROWS = 64


def fold_layer_norm(w: torch.Tensor, gain: torch.Tensor, beta: Optional[torch.Tensor],
                    bias: Optional[torch.Tensor]):
    """Folds a LayerNorm's gain and bias into the bfloat16 matrix that reads it.  Returns
    (w', colsum, bias'): LN(x) w^T + bias = rstd * (x w'^T - mean * colsum) + bias'."""
    _need_cuda(w, gain, beta, bias)
    n_out, k_dim = w.shape
    _need(w.dtype == torch.bfloat16 and w.is_contiguous(), "the matrix must be dense bfloat16")
    _need(gain.dtype == torch.float32 and gain.numel() == k_dim, "gain must be float32 [inner]")
    _need(beta is None or (beta.dtype == torch.float32 and beta.numel() == k_dim), "beta must be float32 [inner]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    w_out = torch.empty_like(w)
    colsum = torch.empty(n_out, dtype=torch.float32, device=w.device)
    bias_out = torch.empty(n_out, dtype=torch.float32, device=w.device)
    with library.unrecorded():
        rc = library.kernels().mgpt_fold_layernorm(_ptr(w), _ptr(gain), _ptr(beta), _ptr(bias), _ptr(w_out),
                                                   _ptr(colsum), _ptr(bias_out), n_out, k_dim, _stream())
    _check(rc, "fold_layer_norm")
    return w_out, colsum, bias_out


def linear_skinny(a: Optional[torch.Tensor], w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  n_rows: int, epilogue: int = EPI_NONE, *, ln_x: Optional[torch.Tensor] = None,
                  ln_colsum: Optional[torch.Tensor] = None, ln_eps: float = 0.0,
                  ln_rows: Optional[torch.Tensor] = None, scatter=None, general_only: bool = False,
                  partials: Optional[torch.Tensor] = None, w_packed: Optional[torch.Tensor] = None,
                  rows_mode: int = 0, rows_per_group: int = 0) -> bool:
    """bfloat16 MFMA product for at most 64 rows.  With ln_x (the float32 residual stream; ln_rows an
    optional gather) the rows are read through a LayerNorm that fold_layer_norm folded into w, bias
    and ln_colsum.  scatter = (k_pool, v_pool, slot_mapping, q_width, kv_width) also stores the new
    keys and values into their pages.  Up to 16 rows with an inner size that is a multiple of 32 go
    to the kernel laid out for a decode step's latency unless general_only is set.  partials:
    float32 scratch of linear_skinny_partials(...) elements, with which a long inner size under many
    rows is split over workgroups.  w_packed: pack_weight(w), which the decode kernel reads faster
    than w itself.  rows_mode: how the decode kernel treats 17 to 64 rows (0: it chooses, ROWS_SHARE_W:
    one workgroup per column tile takes all rows, ROWS_GROUPS: one per column tile and 16 rows); rows_per_group:
    16, 8, 4, 2 or 1 rows to a workgroup of one tile (0: the kernel's launcher chooses).  Returns False, having launched nothing, when the kernel does not take the shape."""
    if n_rows > _SKINNY_MAX_ROWS or w.dtype != torch.bfloat16:
        return False
    n_out, k_dim = w.shape
    if k_dim % 16 != 0:
        return False
    _need_cuda(a, w, bias, out, ln_x, ln_colsum, ln_rows)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    if epilogue == EPI_RESIDUAL:
        _need(out.dtype == torch.float32, "the residual stream is float32")
    elif epilogue in (EPI_GELU, SK_EPI_QKV):
        _need(out.dtype == torch.bfloat16, "this epilogue writes bfloat16")
    lda = 0
    if ln_x is not None:
        _need(ln_x.dtype == torch.float32 and ln_x.is_contiguous() and ln_x.shape[1] == k_dim,
              "the residual stream must be dense float32 rows of the inner size")
        _need(ln_colsum is not None and ln_colsum.dtype == torch.float32 and ln_colsum.numel() == n_out,
              "the folded column sums must be float32 [out]")
        if ln_rows is None:
            _need(ln_x.shape[0] >= n_rows, "too few residual rows")
        else:
            _need_i32("ln_rows", ln_rows, n_rows)
    else:
        if a is None or a.dtype != torch.bfloat16:
            return False
        _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
              "activation must be [>=n_rows, inner] with unit inner stride")
        if a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0:
            return False
        lda = a.stride(0)
    if w_packed is not None:
        _need_cuda(w_packed)
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and k_dim % 32 == 0
              and w_packed.numel() == -(-n_out // 16) * 16 * k_dim and w_packed.data_ptr() % 16 == 0,
              "w_packed must be pack_weight(w)")
    if partials is not None:
        _need_cuda(partials)
        _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0,
              "partials must be contiguous, 16-byte aligned float32")
    kp = vp = sm = None
    q_width = kv_width = head_dim = n_kv_head = page_size = 0
    if epilogue == SK_EPI_QKV:
        kp, vp, sm, q_width, kv_width = scatter
        _need(kp.shape == vp.shape and kp.dim() == 4 and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16,
              "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
        _, n_kv_head, page_size, head_dim = kp.shape
        _need_i32("slot_mapping", sm, n_rows)
    rc = library.kernels().mgpt_linear_skinny(
        _ptr(a if ln_x is None else None), lda, _ptr(ln_x), _ptr(ln_rows), _ptr(ln_colsum),
        float(ln_eps), _ptr(w), _ptr(w_packed), _ptr(bias), _ptr(out), _dtype_code(out), out.stride(0), n_rows,
        n_out, k_dim, epilogue, _ptr(kp), _ptr(vp), _ptr(sm), q_width, kv_width, head_dim, n_kv_head, page_size,
        1 if general_only else rows_mode | (rows_per_group << 8), _ptr(partials), 0 if partials is None else partials.numel(), _stream())
    if rc == -2:
        return False
    _check(rc, "linear_skinny", 2 if partials is not None else 1)
    return True


def pack_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """A copy of a bfloat16 matrix [out, in] in the layout the decode step's product loads in 1 KB
    pieces (blocks of 16 rows x 32 columns in MFMA operand order; rows padded to a multiple of 16
    with zeros).  None if the inner size is no multiple of 32."""
    _need_cuda(w)
    _need(w.dtype == torch.bfloat16 and w.dim() == 2 and w.is_contiguous(), "the matrix must be dense bfloat16")
    n_out, k_dim = w.shape
    if k_dim % 32 != 0 or w.data_ptr() % 16 != 0:
        return None
    packed = torch.empty(-(-n_out // 16) * 16 * k_dim, dtype=torch.bfloat16, device=w.device)
    with library.unrecorded():
        _check(library.kernels().mgpt_pack_weight(_ptr(w), _ptr(packed), n_out, k_dim, _stream()), "pack_weight")
    return packed


ROWS_SHARE_W, ROWS_GROUPS = 2, 3


def linear_head_best(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, n_rows: int,
                     best_val: torch.Tensor, best_idx: torch.Tensor, limit: int,
                     w_packed: Optional[torch.Tensor] = None) -> bool:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias) in float32 for at most 16 bfloat16 rows, and beside it,
    per row and tile of 16 columns, the largest value among the columns below `limit` and its column
    (the lowest among equals): best_val float32, best_idx int32, both [>=n_rows, out / 16].  What
    sample() takes as tile_best.  False, having launched nothing, if the decode kernel does not take
    the shape."""
    n_out, k_dim = w.shape
    if (n_rows > 16 or w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or out.dtype != torch.float32
            or k_dim % 32 or n_out % 16 or a.stride(0) % 8 or a.data_ptr() % 16 or out.stride(0) % 4
            or out.data_ptr() % 16):
        return False
    _need_cuda(a, w, bias, out, best_val, best_idx, w_packed)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out and bias.data_ptr() % 16 == 0),
          "bias must be aligned float32 [out]")
    tiles = n_out // 16
    _need(best_val.dtype == torch.float32 and best_idx.dtype == torch.int32 and best_val.is_contiguous()
          and best_idx.is_contiguous() and tuple(best_val.shape) == tuple(best_idx.shape)
          and best_val.dim() == 2 and best_val.shape[0] >= n_rows and best_val.shape[1] == tiles,
          "best_val and best_idx must be dense float32 / int32 [>=n_rows, out / 16]")
    _need(0 < limit <= n_out, "limit must lie in 1..out")
    if w_packed is not None:
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and w_packed.numel() == n_out * k_dim
              and w_packed.data_ptr() % 16 == 0, "w_packed must be pack_weight(w)")
    rc = library.kernels().mgpt_linear_head_best(
        _ptr(a), a.stride(0), None, None, None, 0.0, _ptr(w), _ptr(w_packed), _ptr(bias), _ptr(out), out.stride(0),
        n_rows, n_out, k_dim, _ptr(best_val), _ptr(best_idx), int(limit), _stream())
    if rc == -2:
        return False
    _check(rc, "linear_head_best")
    return True


def linear_decode_parts(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], partials: torch.Tensor,
                        n_rows: int, w_packed: Optional[torch.Tensor] = None) -> int:
    """The split product's first half alone: partials[p, :n_rows] (float32 [parts, n_rows, out], dense)
    = a[:n_rows] @ w[:, stretch p of the inner size].T, the first with the bias added; nobody adds them
    up.  Returns the number of parts, or 0, having launched nothing, for a shape that linear_skinny
    would not split (linear_skinny_partials(n_rows, out, inner, False, EPI_RESIDUAL) == 0)."""
    n_out, k_dim = w.shape
    if (w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or a.stride(0) % 8 or a.data_ptr() % 16
            or not linear_skinny_partials(n_rows, n_out, k_dim, False, EPI_RESIDUAL)):
        return 0
    parts = int(library.kernels().mgpt_linear_decode_parts_count())
    _need_cuda(a, w, bias, partials, w_packed)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out and bias.data_ptr() % 16 == 0),
          "bias must be aligned float32 [out]")
    _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0
          and tuple(partials.shape) == (parts, n_rows, n_out), f"partials must be dense float32 [{parts}, n_rows, out]")
    if w_packed is not None:
        _need(w_packed.dtype == torch.bfloat16 and w_packed.is_contiguous() and w_packed.numel() == n_out * k_dim
              and w_packed.data_ptr() % 16 == 0, "w_packed must be pack_weight(w)")
    rc = library.kernels().mgpt_linear_decode_parts(_ptr(a), a.stride(0), _ptr(w), _ptr(w_packed), _ptr(bias),
                                                    _ptr(partials), n_rows, n_out, k_dim, _stream())
    if rc == -2:
        return 0
    _check(rc, "linear_decode_parts")
    return parts


def linear_skinny_row_groups(n_rows: int, n_out: int, k_dim: int) -> bool:
    """Whether linear_skinny, left to choose, gives every 16 of these rows workgroups of their own
    (a folded LayerNorm then costs a workgroup what it costs at 16 rows)."""
    return bool(library.kernels().mgpt_linear_skinny_row_groups(n_rows, n_out, k_dim))


def linear_skinny_partials(n_rows: int, n_out: int, k_dim: int, has_ln: bool, epilogue: int) -> int:
    """float32 elements of scratch with which linear_skinny would split this shape's inner size over
    workgroups; 0 if it would not."""
    return int(library.kernels().mgpt_linear_skinny_partials(n_rows, n_out, k_dim, 1 if has_ln else 0, epilogue))


def paged_attention_split_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                               block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor,
                               q_req: torch.Tensor, n_tokens: int, n_req: int, n_head: int, scale: float,
                               window: int = 0, fast: bool = True) -> bool:
    """bfloat16 attention with each (token, head)'s keys split over four waves.  False if refused.
    fast=False keeps to the variant that takes every head size."""
    if q.dtype != torch.bfloat16:
        return False
    n_kv_head, page_size, head_dim = _check_attention_args(
        q, out, k_pool, v_pool, block_tables, cu_q, seq_lens, q_req, n_tokens, n_req, n_head)
    if head_dim % 8 != 0 or head_dim > 256 or k_pool.data_ptr() % 16 != 0:
        return False
    fn = library.kernels().mgpt_paged_attention_split_bf16
    if fast and head_dim in (16, 32, 64, 128) and q.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0:
        fn = library.kernels().mgpt_paged_attention_split_fast_bf16   # all loads 16 bytes wide
    rc = fn(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), _ptr(q_req), n_tokens, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), _stream())
    if rc == -2:
        return False
    _check(rc, "paged_attention_split_bf16")
    return True


def paged_attention_decode_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                                block_tables: torch.Tensor, positions: torch.Tensor, q_req: torch.Tensor,
                                n_tokens: int, n_head: int, scale: float, window: int = 0,
                                identity: bool = False, cu_q: Optional[torch.Tensor] = None) -> bool:
    """bfloat16 attention for single tokens (one query per request and step), keys split over eight
    waves.  positions[n] is token n's absolute position, q_req[n] its block table row or -1 for a
    padded token; identity=True promises q_req[n] in (n, -1).  With cu_q (the requests' token offsets;
    not with identity) tokens of requests that bring more than one token are skipped.  False if
    refused (other head sizes than 16, 32, 64, 128)."""
    if q.dtype != torch.bfloat16:
        return False
    _need_cuda(q, out, k_pool, v_pool, block_tables, positions, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous()
          and k_pool.dtype == torch.bfloat16 and v_pool.dtype == torch.bfloat16,
          "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
    num_pages, n_kv_head, page_size, head_dim = k_pool.shape
    if head_dim not in (16, 32, 64, 128) or q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0 \
            or k_pool.data_ptr() % 16 != 0 or v_pool.data_ptr() % 16 != 0:
        return False
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[0] >= n_tokens and q.shape[1] >= n_head * head_dim,
          "q must be [>=n_tokens, >=heads*head_dim] with unit inner stride")
    _need(out.dtype == torch.bfloat16 and out.dim() == 2 and out.stride(1) == 1 and out.shape[0] >= n_tokens
          and out.shape[1] >= n_head * head_dim, "out must be bfloat16 [>=n_tokens, >=heads*head_dim]")
    _need(n_head % n_kv_head == 0, "query heads must be a multiple of key/value heads")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "block_tables must be dense int32 [requests, blocks]")
    _need_i32("positions", positions, n_tokens)
    _need_i32("q_req", q_req, n_tokens)
    if identity:
        _need(block_tables.shape[0] >= n_tokens, "a decode-only step needs a block table row per token")
        _need(cu_q is None, "cu_q is for steps that are not decode-only")
    if cu_q is not None:
        _need_cuda(cu_q)
        _need_i32("cu_q", cu_q, block_tables.shape[0] + 1)
    rc = library.kernels().mgpt_paged_attention_decode_bf16(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(positions), _ptr(q_req), _ptr(cu_q), n_tokens, n_head, n_kv_head, head_dim, page_size,
        num_pages, float(scale), int(window), 1 if identity else 0, _stream())
    if rc == -2:
        return False
    _check(rc, "paged_attention_decode_bf16")
    return True


_MFMA_PARTIALS: dict = {}   # the library's answer per size: asked at every product of every step


def linear_mfma_partials(n_rows: int, n_out: int, k_dim: int, epilogue: int) -> int:
    """Floats of scratch that linear_mfma would use to split this product along its inner size
    (0: it would not split it)."""
    key = (n_rows, n_out, k_dim, epilogue)
    hit = _MFMA_PARTIALS.get(key)
    if hit is None:
        if len(_MFMA_PARTIALS) > 4096:
            _MFMA_PARTIALS.clear()
        hit = _MFMA_PARTIALS[key] = int(library.kernels().mgpt_linear_mfma_partials(n_rows, n_out, k_dim, epilogue))
    return hit


def linear_mfma_parts(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], partials: torch.Tensor,
                      n_rows: int) -> bool:
    """The tiled product's first half alone where it splits the inner size: partials[p, :n_rows]
    (float32 [parts, n_rows, out], dense, parts = linear_mfma_partials(n_rows, out, inner, EPI_RESIDUAL)
    // (n_rows * out)) = a[:n_rows] @ w[:, stretch p].T, the first with the bias added; nobody adds
    them up.  False, having launched nothing, where the product would not be split."""
    n_out, k_dim = w.shape
    need = linear_mfma_partials(n_rows, n_out, k_dim, EPI_RESIDUAL)
    if (not need or w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16 or a.stride(0) % 8 or a.data_ptr() % 16
            or w.data_ptr() % 16 or k_dim % 16):
        return False
    parts = need // (n_rows * n_out)
    _need_cuda(a, w, bias, partials)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    _need(partials.dtype == torch.float32 and partials.is_contiguous() and partials.data_ptr() % 16 == 0
          and tuple(partials.shape) == (parts, n_rows, n_out), f"partials must be dense float32 [{parts}, n_rows, out]")
    rc = library.kernels().mgpt_linear_mfma_parts(_ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(partials),
                                                  partials.numel(), n_rows, n_out, k_dim, _stream())
    if rc == -2:
        return False
    _check(rc, "linear_mfma_parts")
    return True


def linear_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                n_rows: int, epilogue: int, scatter=None, shape: Optional[int] = None,
                partials: Optional[torch.Tensor] = None, k_parts: Optional[int] = None) -> bool:
    """Tiled bfloat16 MFMA product for many rows.  scatter = (k_pool, v_pool, slot_mapping, q_width,
    kv_width) also stores the new keys and values into their pages (bfloat16 output, no other
    epilogue).  `partials`: float32 scratch with which a long inner size over few tiles is split
    among workgroups (linear_mfma_partials says how much it takes).  `shape` (0 = 256 x 256 tiles,
    1 = 128 x 256, 2 = 128 x 64, 3 = 64 x 64, 4 = 32 x 32, 5 and 6 = 64 x 64 and 32 x 32 with four
    steps on their way from memory, 7 = 64 x 64 with two wave groups that share a tile, float32 outputs, 8 to 12 = operand slices straight
    into LDS with tiles of 32 x 32, 64 x 64, 128 x 64, 128 x 192, 32 x 32 with six stages: an inner size that is a
    multiple of 64) and
    `k_parts` fix what the library otherwise chooses by the size.  False when it does not take the shape."""
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return False
    n_out, k_dim = w.shape
    if k_dim % 16 != 0 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0 or w.data_ptr() % 16 != 0:
        return False
    if scatter is not None and (epilogue != EPI_NONE or out.dtype != torch.bfloat16):
        return False
    if (epilogue, out.dtype) not in ((EPI_NONE, torch.bfloat16), (EPI_NONE, torch.float32),
                                     (EPI_GELU, torch.bfloat16), (EPI_RESIDUAL, torch.float32)):
        return False
    _need_cuda(a, w, bias, out)
    _need(w.is_contiguous(), "weight must be dense [out, in]")
    _need(a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k_dim and a.shape[0] >= n_rows,
          "activation must be [>=n_rows, inner] with unit inner stride")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_out and out.shape[0] >= n_rows,
          "output must be [>=n_rows, >=out] with unit inner stride")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_out), "bias must be float32 [out]")
    if scatter is not None:
        kp, vp, sm, q_width, kv_width = scatter
        _need_cuda(kp, vp, sm)
        _need(kp.shape == vp.shape and kp.dim() == 4 and kp.is_contiguous() and vp.is_contiguous()
              and kp.dtype == torch.bfloat16 and vp.dtype == torch.bfloat16,
              "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
        _, n_kv_head, page_size, head_dim = kp.shape
        _need_i32("slot_mapping", sm, n_rows)
        rc = library.kernels().mgpt_linear_mfma_qkv(
            _ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(out), out.stride(0), n_rows, n_out, k_dim, _ptr(kp),
            _ptr(vp), _ptr(sm), q_width, kv_width, head_dim, n_kv_head, page_size, -1 if shape is None else int(shape),
            _stream())
    else:
        if partials is not None:
            _need_cuda(partials)
            _need(partials.dtype == torch.float32 and partials.is_contiguous(), "partials must be dense float32")
        args = (_ptr(a), a.stride(0), _ptr(w), _ptr(bias), _ptr(out), _dtype_code(out), out.stride(0), n_rows,
                n_out, k_dim, epilogue, _ptr(partials), 0 if partials is None else partials.numel(), _stream())
        if shape is None and k_parts is None:
            rc = library.kernels().mgpt_linear_mfma(*args)
        else:
            rc = library.kernels().mgpt_linear_mfma_shape(-1 if shape is None else int(shape),
                                                          0 if k_parts is None else int(k_parts), *args)
    if rc == -2:
        return False
    _check(rc, "linear_mfma", 2 if partials is not None else 1)
    return True


def prefill_attention_bf16(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                           block_tables: torch.Tensor, cu_q: torch.Tensor, seq_lens: torch.Tensor, n_req: int,
                           max_q_len: int, n_head: int, scale: float, window: int = 0,
                           single_below: int = 0) -> bool:
    """MFMA tile attention for steps with prompt portions (every request's tokens are consecutive
    rows of q from cu_q; a request may bring none).  Requests that bring exactly one token, and that
    among the step's first `single_below` tokens, are left to another kernel.  False when it does
    not take the case."""
    if q.dtype != torch.bfloat16:
        return False
    _need_cuda(q, out, k_pool, v_pool, block_tables, cu_q, seq_lens)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous(),
          "key and value pools must be dense [pages, kv_heads, page_size, head_dim]")
    _, n_kv_head, page_size, head_dim = k_pool.shape
    if head_dim not in (32, 64, 96, 128) or q.stride(0) % 8 != 0 or q.data_ptr() % 16 != 0 \
            or k_pool.data_ptr() % 16 != 0 or v_pool.data_ptr() % 16 != 0:
        return False
    _need(q.dtype == out.dtype == k_pool.dtype == v_pool.dtype, "queries, output and pools must share a dtype")
    _need(q.stride(1) == 1 and out.stride(1) == 1, "query and output rows must have unit inner stride")
    _need(q.shape[1] >= n_head * head_dim and out.shape[1] >= n_head * head_dim,
          "query/output rows are narrower than n_head * head_dim")
    _need(n_head % n_kv_head == 0, "n_head must be a multiple of the number of key/value heads")
    _need(block_tables.dim() == 2 and block_tables.dtype == torch.int32 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_req, "block_tables must be dense int32 [>=requests, max_blocks]")
    _need_i32("cu_q", cu_q, n_req + 1)
    _need_i32("seq_lens", seq_lens, n_req)
    rc = library.kernels().mgpt_prefill_attention_bf16(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(block_tables),
        block_tables.shape[1], _ptr(cu_q), _ptr(seq_lens), n_req, max_q_len, n_head, n_kv_head, head_dim,
        page_size, float(scale), int(window), int(single_below), _stream())
    if rc == -2:
        return False
    _check(rc, "prefill_attention_bf16")
    return True


# ---------------------------------------------------------------- decode steps of few rows, fused
FUSED_MAX_WIDTH = 512
FUSED_MLP_SLICE = 64


def fused_parts_limit(width: int) -> int:
    """Most pending sums of a residual of this width that the fused kernels add up on their way in
    (0: they do not take the width)."""
    if width <= 0 or width % 32 or width > FUSED_MAX_WIDTH:
        return 0
    return int(library.kernels().mgpt_fused_parts_limit(width))


def _residual_args(pending, width: int):
    """The argument block of a residual that is still a sum (ops.residual.PendingSums)."""
    base, partials, n_parts = pending.base, pending.partials, pending.n_parts
    tok = pos = ids = positions = None
    if base is None:
        tok, pos, ids, positions = pending.tables
        _need_cuda(tok, pos, ids, positions)
        _need(tok.dtype == torch.bfloat16 and tok.is_contiguous() and tok.shape[1] == width,
              "the token table must be dense bfloat16 [vocab, width]")
        _need(pos is None or (pos.dtype == torch.bfloat16 and pos.is_contiguous() and pos.shape[1] == width),
              "the position table must be dense bfloat16 [positions, width]")
    else:
        _need_cuda(base)
        _need(base.dtype == torch.float32 and base.is_contiguous() and base.shape[1] == width,
              "the residual rows must be dense float32 [rows, width]")
    stride = 0
    if n_parts:
        _need_cuda(partials)
        _need(partials.dtype == torch.float32 and partials.dim() == 3 and partials.is_contiguous()
              and partials.shape[0] >= n_parts and partials.shape[2] == width,
              "pending sums must be dense float32 [parts, rows, width]")
        stride = partials.stride(0)
    return (_ptr(base), _ptr(partials) if n_parts else None, n_parts, stride, _ptr(tok), _ptr(pos), _ptr(ids),
            _ptr(positions))


def _overlap(a: Optional[torch.Tensor], b: Optional[torch.Tensor]) -> bool:
    """Whether two tensors' bytes overlap."""
    if a is None or b is None or not a.numel() or not b.numel():
        return False
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def _residual_rows(pending) -> int:
    """Rows that every array of a pending residual holds."""
    rows = 1 << 30
    if pending.base is not None:
        rows = min(rows, pending.base.shape[0])
    else:
        rows = min(rows, pending.tables[2].numel())
    if pending.n_parts:
        rows = min(rows, pending.partials.shape[1])
    return rows


def fused_attention_tokens(n_rows: int, n_head: int, head_dim: int) -> int:
    """Tokens that a workgroup of fused_attention_decode takes in a step of n_rows rows.  With more
    than one, rows that are no table rows must be handed over normed; 0: the kernel does not take so
    many rows."""
    return int(library.kernels().mgpt_fused_attention_tokens(int(n_rows), int(n_head), int(head_dim)))


def fused_attention_decode(pending, settled: Optional[torch.Tensor], gain: torch.Tensor, beta: Optional[torch.Tensor],
                           eps: float, wqkv_packed: torch.Tensor, bqkv: Optional[torch.Tensor],
                           wproj_packed: torch.Tensor, bproj: Optional[torch.Tensor], out_partials: torch.Tensor,
                           k_pool: torch.Tensor, v_pool: torch.Tensor, slot_mapping: torch.Tensor,
                           block_tables: torch.Tensor, positions: torch.Tensor, q_req: torch.Tensor, n_rows: int,
                           n_head: int, scale: float, normed: Optional[torch.Tensor] = None) -> bool:
    """LayerNorm, one head's q/k/v, cache write, attention and that head's share of the output
    projection, for the single tokens of a decode-only step: out_partials[h, n] is head h's share
    of what token n adds to the residual.  The residual comes as a sum (pending), whose value is
    stored to `settled` on the way.  In a step of so many rows that a workgroup takes several
    tokens (fused_attention_tokens), rows that are no table rows come normed instead (`normed`:
    bfloat16 [rows, width], the LayerNorm of the plain rows `pending.base`; nothing is stored to
    `settled`, which may be None).  False, having launched nothing, if the kernel does not take the
    shape."""
    width = gain.numel()
    _need_cuda(settled, gain, beta, wqkv_packed, bqkv, wproj_packed, bproj, out_partials, k_pool, v_pool,
               slot_mapping, block_tables, positions, q_req)
    _need(k_pool.shape == v_pool.shape and k_pool.dim() == 4 and k_pool.is_contiguous() and v_pool.is_contiguous()
          and k_pool.dtype == torch.bfloat16 and v_pool.dtype == torch.bfloat16,
          "key and value pools must be dense bfloat16 [pages, kv_heads, page_size, head_dim]")
    num_pages, n_kv_head, page_size, head_dim = k_pool.shape
    q_width = n_head * head_dim
    if (n_kv_head != n_head or head_dim not in (16, 32, 64, 128) or width % 32 or width > FUSED_MAX_WIDTH
            or q_width % 32 or page_size & (page_size - 1) or pending.n_parts > fused_parts_limit(width)):
        return False
    tokens = fused_attention_tokens(n_rows, n_head, head_dim)
    use_normed = pending.base is not None and tokens > 1
    if tokens == 0 or (use_normed and (normed is None or pending.n_parts)):
        return False
    args = _residual_args(pending, width)
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than the step")
    if use_normed:
        _need_cuda(normed)
        _need(normed.dtype == torch.bfloat16 and normed.is_contiguous() and normed.dim() == 2
              and normed.shape[1] == width and normed.shape[0] >= n_rows, "normed rows must be dense bfloat16 [>=rows, width]")
    else:
        _need(settled is not None and settled.dtype == torch.float32 and settled.is_contiguous()
              and settled.shape[1] == width and settled.shape[0] >= n_rows
              and (pending.base is None or settled.data_ptr() != pending.base.data_ptr()),
              "the settled rows need a dense float32 array of their own")
    for name, t, numel in (("gain", gain, width), ("beta", beta, width), ("qkv bias", bqkv, 3 * q_width),
                           ("projection bias", bproj, width)):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == numel), f"{name} must be float32 [{numel}]")
    _need(wqkv_packed.dtype == torch.bfloat16 and wqkv_packed.numel() == 3 * q_width * width,
          "wqkv_packed must be pack_weight of the [3 * heads * head_dim, width] matrix")
    _need(wproj_packed.dtype == torch.bfloat16 and wproj_packed.numel() == width * q_width,
          "wproj_packed must be pack_weight of the [width, heads * head_dim] matrix")
    _need(out_partials.dtype == torch.float32 and out_partials.dim() == 3 and out_partials.is_contiguous()
          and out_partials.shape[0] >= n_head and out_partials.shape[1] >= n_rows and out_partials.shape[2] == width,
          "out_partials must be dense float32 [>=heads, >=rows, width]")
    # a workgroup adds the pending sums up while others of the launch already store theirs
    _need(not (pending.n_parts and _overlap(out_partials, pending.partials)),
          "out_partials must not be the array that holds the pending sums")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
          and block_tables.shape[0] >= n_rows, "block_tables must be dense int32 [>=rows, blocks]")
    _need_i32("slot_mapping", slot_mapping, n_rows)
    _need_i32("positions", positions, n_rows)
    _need_i32("q_req", q_req, n_rows)
    rc = library.kernels().mgpt_fused_attention_decode(
        *args, None if use_normed else _ptr(settled), _ptr(normed) if use_normed else None, _ptr(gain), _ptr(beta),
        float(eps), _ptr(wqkv_packed), _ptr(bqkv), _ptr(wproj_packed),
        _ptr(bproj), _ptr(out_partials), out_partials.stride(0), _ptr(k_pool), _ptr(v_pool), _ptr(slot_mapping),
        _ptr(block_tables), block_tables.shape[1], _ptr(positions), _ptr(q_req), n_rows, width, n_head, head_dim,
        page_size, num_pages, float(scale), _stream())
    if rc == -2:
        return False
    _check(rc, "fused_attention_decode")
    return True


def fused_mlp_parts(hidden: int) -> int:
    """Parts that fused_mlp_decode leaves of its output (0: it does not take this hidden size)."""
    return hidden // FUSED_MLP_SLICE if hidden > 0 and hidden % FUSED_MLP_SLICE == 0 else 0


def fused_mlp_decode(pending, settled: torch.Tensor, gain: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
                     wfc_packed: torch.Tensor, bfc: Optional[torch.Tensor], wproj_packed: torch.Tensor,
                     bproj: Optional[torch.Tensor], out_partials: torch.Tensor, n_rows: int, hidden: int) -> bool:
    """LayerNorm, 64 hidden units of the first product with bias and GELU-tanh, and their share of
    the second product, per workgroup: out_partials[j, n] is what hidden units 64 j .. add to row n
    of the residual.  False, having launched nothing, if the kernel does not take the shape."""
    width = gain.numel()
    parts = fused_mlp_parts(hidden)
    if not parts or width % 32 or width > FUSED_MAX_WIDTH or pending.base is None \
            or pending.n_parts > fused_parts_limit(width):
        return False
    _need_cuda(settled, gain, beta, wfc_packed, bfc, wproj_packed, bproj, out_partials)
    args = _residual_args(pending, width)
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than the step")
    _need(settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[1] == width
          and settled.shape[0] >= n_rows and (pending.base is None or settled.data_ptr() != pending.base.data_ptr()),
          "the settled rows need a dense float32 array of their own")
    for name, t, numel in (("gain", gain, width), ("beta", beta, width), ("first bias", bfc, hidden),
                           ("second bias", bproj, width)):
        _need(t is None or (t.dtype == torch.float32 and t.numel() == numel), f"{name} must be float32 [{numel}]")
    _need(wfc_packed.dtype == torch.bfloat16 and wfc_packed.numel() == hidden * width
          and wproj_packed.dtype == torch.bfloat16 and wproj_packed.numel() == hidden * width,
          "the matrices must be pack_weight of [hidden, width] and [width, hidden]")
    _need(out_partials.dtype == torch.float32 and out_partials.dim() == 3 and out_partials.is_contiguous()
          and out_partials.shape[0] >= parts and out_partials.shape[1] >= n_rows and out_partials.shape[2] == width,
          "out_partials must be dense float32 [>=hidden/64, >=rows, width]")
    _need(not (pending.n_parts and _overlap(out_partials, pending.partials)),
          "out_partials must not be the array that holds the pending sums")
    rc = library.kernels().mgpt_fused_mlp_decode(
        *args, _ptr(settled), _ptr(gain), _ptr(beta), float(eps), _ptr(wfc_packed), _ptr(bfc), _ptr(wproj_packed),
        _ptr(bproj), _ptr(out_partials), out_partials.stride(0), n_rows, width, hidden, _stream())
    if rc == -2:
        return False
    _check(rc, "fused_mlp_decode")
    return True


RESIDUAL_MAX_WIDTH = 4096
_RESIDUAL_PARTS_LIMIT: Dict[int, int] = {}


def residual_parts_limit(width: int) -> int:
    """Most parts of a pending residual of this width that residual_layer_norm adds up (0: the width
    is not taken).  Wider than the fused kernels take: a row up to RESIDUAL_MAX_WIDTH."""
    hit = _RESIDUAL_PARTS_LIMIT.get(width)
    if hit is None:
        hit = _RESIDUAL_PARTS_LIMIT[width] = int(library.kernels().mgpt_residual_parts_limit(int(width)))
    return hit


def residual_layer_norm(pending, gain: torch.Tensor, beta: Optional[torch.Tensor], eps: float,
                        rows: Optional[torch.Tensor], out: torch.Tensor, n_rows: int,
                        settled: Optional[torch.Tensor] = None) -> bool:
    """out[i] = LayerNorm of row rows[i] (or i) of a residual that is still a sum.  With `settled`
    (float32 rows; may be the sum's base itself) the rows' sums are stored there too.  False if
    the width is not taken."""
    width = gain.numel()
    if width % 32 or width > RESIDUAL_MAX_WIDTH or pending.base is None or pending.n_parts > residual_parts_limit(width):
        return False
    _need_cuda(gain, beta, rows, out, settled)
    _need(settled is None or (settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[1] == width
                              and settled.shape[0] >= (n_rows if rows is None else 0) and settled.data_ptr() % 16 == 0),
          "the settled rows must be dense float32 of the residual's width")
    _need(settled is None or rows is None, "settling through a row gather is not supported")
    args = _residual_args(pending, width)
    _need(gain.dtype == torch.float32 and (beta is None or (beta.dtype == torch.float32 and beta.numel() == width)),
          "gain and beta must be float32 [width]")
    _need(out.is_contiguous() and out.shape[1] == width and out.shape[0] >= n_rows, "LayerNorm output too small")
    if rows is None:
        _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than asked for")
    else:
        _need_i32("rows", rows, n_rows)
    rc = library.kernels().mgpt_residual_layernorm(*args, _ptr(gain), _ptr(beta), float(eps), _ptr(rows), _ptr(out),
                                                   _dtype_code(out), n_rows, width, _ptr(settled), _stream())
    if rc == -2:
        return False
    _check(rc, "residual_layer_norm")
    return True


def residual_settle(pending, settled: torch.Tensor, n_rows: int) -> bool:
    """settled[:n_rows] = the rows of a residual that is still a sum (settled may be its base).
    False if the width is not taken."""
    width = settled.shape[1]
    if width % 32 or width > RESIDUAL_MAX_WIDTH or pending.base is None:
        return False
    _need_cuda(settled)
    args = _residual_args(pending, width)
    _need(settled.dtype == torch.float32 and settled.is_contiguous() and settled.shape[0] >= n_rows,
          "the settled rows must be dense float32")
    _need(_residual_rows(pending) >= n_rows, "the pending residual holds fewer rows than asked for")
    rc = library.kernels().mgpt_residual_settle(*args, _ptr(settled), n_rows, width, _stream())
    if rc == -2:
        return False
    _check(rc, "residual_settle")
    return True
