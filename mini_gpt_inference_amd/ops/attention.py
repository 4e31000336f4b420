"""Chooses the attention kernel for a step."""

from __future__ import annotations

import torch

from . import kernels


def _mixed_step(ctx, q, out, k_pool, v_pool, group, n_head: int, scale: float, window: int) -> bool:
    """A step with prompt portions.  The requests that lead the step with one token each (a scheduler
    puts the decoding requests first) go to the decode kernel, token n being request n; the rest,
    prompt portions mostly, to the MFMA tile kernel, which would spend a 64-query tile on a single
    token.  False, having launched nothing, if the tile kernel does not take the case."""
    q_lens = ctx.host_q_lens
    lead = 0
    if q_lens is not None:
        while lead < len(q_lens) and q_lens[lead] == 1:
            lead += 1
    rest = ctx.n_req - lead
    if lead and rest and kernels.prefill_attention_bf16(
            q, out, k_pool, v_pool, group.block_tables[lead:], ctx.cu_q[lead:], ctx.seq_lens[lead:], rest,
            ctx.max_q_len, n_head, scale, window):
        if kernels.paged_attention_decode_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.positions, ctx.q_req,
                                               lead, n_head, scale, window, identity=True):
            return True
        # the decode kernel refuses this head or page size: the tile kernel for the leading requests too
        return kernels.prefill_attention_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                              lead, 1, n_head, scale, window)
    return kernels.prefill_attention_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                          ctx.n_req, ctx.max_q_len, n_head, scale, window)


def _padded_mixed_step(ctx, q, out, k_pool, v_pool, group, n_head: int, scale: float, window: int) -> bool:
    """A step with prompt portions that is padded to its bucket's sizes (a graph replays it for every
    step of the bucket): which request brings how many tokens is known on the device only.  The
    decode kernel goes over the step's first `ctx.lead_cap` tokens (decoding requests lead a step)
    and leaves out those of requests with several tokens; the tile kernel goes over all requests and
    leaves out those whose one token the decode kernel had; requests and tokens of the padding have
    neither.  False if the tile kernel refuses (the caller's general kernel then does all tokens again)."""
    r = ctx.cu_q.numel() - 1
    lead = min(ctx.lead_cap, ctx.n_rows)
    singles = lead > 0 and kernels.paged_attention_decode_bf16(
        q, out, k_pool, v_pool, group.block_tables, ctx.positions, ctx.q_req, lead, n_head, scale, window,
        cu_q=ctx.cu_q)
    return kernels.prefill_attention_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens, r,
                                          ctx.n_rows, n_head, scale, window, single_below=lead if singles else 0)


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
        if not ctx.decode_only and not ctx.padded and _mixed_step(ctx, q, out, k_pool, v_pool, group, n_head, scale,
                                                                  window):
            return
        if not ctx.decode_only and ctx.padded and _padded_mixed_step(ctx, q, out, k_pool, v_pool, group, n_head,
                                                                     scale, window):
            return
        if kernels.paged_attention_split_bf16(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                              ctx.q_req, n, r, n_head, scale, window):
            return
    kernels.paged_attention_generic(q, out, k_pool, v_pool, group.block_tables, ctx.cu_q, ctx.seq_lens,
                                    ctx.q_req, n, r, n_head, scale, window, fast_exp=not ctx.exact)
