"""Chooses the attention kernel for a step."""

from __future__ import annotations

import torch

from . import kernels


def paged_attention(ctx, q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                    group, n_head: int, scale: float, window: int) -> None:
    """Attention of the step's tokens (rows of q) over their requests' pages.

    On the bfloat16 path a decode-only step (token n is request n's one token) uses the kernel
    laid out for a decode step's latency, steps with prompt portions the MFMA tile kernel and the
    rest the kernel that splits a query's keys over four waves; the 32-bit path and every shape
    those refuse use the general kernel, whose order of sums depends only on a query's position."""
    n, r = ctx.n_rows, ctx.cu_q.numel() - 1
    if q.dtype == torch.bfloat16 and not ctx.exact:
        if ctx.decode_only and kernels.paged_attention_decode_bf16(
                q, out, k_pool, v_pool, group.block_tables, ctx.positions, ctx.q_req, n, n_head, scale, window,
                identity=True):
            return
        if not ctx.decode_only and ctx.n_rows == ctx.n_tokens and kernels.prefill_attention_bf16(
                q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens, ctx.n_req, ctx.max_q_len,
                n_head, scale, window):
            return
        if kernels.paged_attention_split_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                              ctx.q_req, n, r, n_head, scale, window):
            return
    kernels.paged_attention_generic(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                    ctx.q_req, n, r, n_head, scale, window, fast_exp=not ctx.exact)
