"""Sequence mixers.  A mixer adds its output into the residual stream."""

from __future__ import annotations

from typing import Dict, Optional, Union

import torch

from ..ops import attention as attention_ops
from ..ops import kernels, residual
from ..ops.linear import LazyNorm, linear, linear_add, packed_weight, plain_residual
from .base import (CacheBinding, KVNeed, MATRIX, Part, StateNeed, StepContext, VECTOR, WeightRequest,
                   register_mixer)
from .positions import PositionEncoding


class Mixer(Part):
    category = "mixer"

    def cache_need(self) -> Union[KVNeed, StateNeed, None]:
        return None

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        """x[:n_rows] += mixer(h[:n_rows]).  x is the float32 residual stream; h is the normed input,
        either a tensor in the compute dtype or an ops.linear.LazyNorm, which linear() takes as it
        is and as_tensor(ctx, h) turns into a tensor."""
        raise NotImplementedError


@register_mixer("paged_causal_attention")
class PagedCausalAttention(Mixer):
    """Multi-head causal self-attention over the paged cache.

    qkv = h Wqkv^T (+ b); q = columns [0, H*D), k = the next Hkv*D, v = the last Hkv*D, head i of
    each = columns i*D..(i+1)*D (reference: src/minigpt_infer/model.py:43,49-53).  New keys and
    values are stored unscaled before attention reads everything up to and including them
    (model.py:55-59).  S = q k^T * scale with scale = 1/sqrt(D) unless given (SDPA's default,
    model.py:87); a query sees the keys of its own request at positions <= its own (and, with a
    window, only the last `window` of them); softmax in float32; y = P v; heads concatenated
    head-major; out = y Wproj^T (+ b) (model.py:89-90), added into the residual (model.py:113)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True

    def __init__(self, width: int, n_head: int, head_dim: int, bias: bool, n_kv_head: Optional[int] = None,
                 scale: Optional[float] = None, window: int = 0) -> None:
        self.width, self.n_head, self.head_dim = int(width), int(n_head), int(head_dim)
        self.n_kv_head = int(n_kv_head) if n_kv_head is not None else self.n_head
        self.has_bias = bool(bias)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.window = int(window)
        if not 0 < self.head_dim <= 256:
            raise ValueError(f"head size {self.head_dim}: the kernels take head sizes up to 256")
        if self.n_head % self.n_kv_head != 0:
            raise ValueError("n_head must be a multiple of n_kv_head")
        self.q_width = self.n_head * self.head_dim
        self.kv_width = self.n_kv_head * self.head_dim
        self.qkv_weight = self.qkv_bias = self.proj_weight = self.proj_bias = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        total = self.q_width + 2 * self.kv_width
        req = {"qkv_weight": WeightRequest((total, self.width), MATRIX),
               "proj_weight": WeightRequest((self.width, self.q_width), MATRIX)}
        if self.has_bias:
            req["qkv_bias"] = WeightRequest((total,), VECTOR)
            req["proj_bias"] = WeightRequest((self.width,), VECTOR)
        return req

    def cache_need(self) -> KVNeed:
        return KVNeed(self.n_kv_head, self.head_dim, self.window)

    def _forward_add_fused(self, ctx: StepContext, h, x: torch.Tensor, binding: CacheBinding,
                           position: PositionEncoding) -> bool:
        """A decode-only step of few rows: one kernel from the residual (as the kernels before left
        it: a sum) through LayerNorm, projections, cache write and attention to this mixer's
        addition to the residual, left as one partial sum per head.  False where that kernel does
        not apply (with nothing launched but, in a step of many rows, the LayerNorm that the other
        path needs as well)."""
        if not (isinstance(h, LazyNorm) and h._tensor is None and h.rows is None and h.x is x
                and getattr(h.norm, "fusable_layer_norm", False) and residual.usable(ctx, self.width, self.n_head)
                and binding.writes and not position.rotates and self.window == 0
                and self.n_kv_head == self.n_head and self.qkv_weight.dtype == torch.bfloat16
                and self.proj_weight.dtype == torch.bfloat16):
            return False
        wqkv, wproj = packed_weight(self.qkv_weight, ctx), packed_weight(self.proj_weight, ctx)
        if wqkv is None or wproj is None:
            return False
        n = ctx.n_rows
        group = ctx.groups[binding.group]
        # In a step of so many rows that a workgroup takes several tokens, every head's workgroup
        # adding up its tokens' pending parts would be most of the kernel's traffic: the LayerNorm
        # kernel adds them up once (x is plain after it) and hands the rows over normed.
        normed = None
        table_rows = ctx.pending is not None and ctx.pending.base is None
        tokens = kernels.fused_attention_tokens(n, self.n_head, self.head_dim)
        if tokens == 0:
            return False
        if not table_rows and tokens > 1:
            normed = h.tensor(ctx)
            if ctx.pending is not None:
                return False
        pending, settled = residual.take(ctx, x)
        parts = residual.parts_buffer(ctx, "attention_parts", self.n_head, n, self.width)
        if not kernels.fused_attention_decode(
                pending, settled, h.norm.weight, h.norm.bias, h.norm.eps, wqkv, self.qkv_bias, wproj, self.proj_bias,
                parts, group.k_pools[binding.index], group.v_pools[binding.index], group.slot_mapping,
                group.block_tables, ctx.positions, ctx.q_req, n, self.n_head, self.scale, normed=normed):
            return False
        ctx.pending = residual.PendingSums(x if normed is not None else settled, parts, self.n_head)
        return True

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, binding: CacheBinding,
                    position: PositionEncoding) -> None:
        if self._forward_add_fused(ctx, h, x, binding, position):
            return
        plain_residual(ctx, h, x)
        n = ctx.n_rows
        total = self.q_width + 2 * self.kv_width
        qkv = ctx.workspace.get("qkv", n, total, ctx.dtype)
        group = ctx.groups[binding.group]
        k_pool, v_pool = group.k_pools[binding.index], group.v_pools[binding.index]
        # a position encoding that rotates queries and keys must act before the keys are stored;
        # only without one may the projection kernel store them itself
        scatter = None
        if binding.writes and not position.rotates:
            scatter = (k_pool, v_pool, group.slot_mapping, self.q_width, self.kv_width)
        stored = linear(ctx, h, self.qkv_weight, self.qkv_bias, qkv, n, scatter=scatter)
        position.rotate(ctx, qkv[:, :self.q_width], qkv[:, self.q_width:self.q_width + self.kv_width], n)
        if binding.writes and not stored:
            kernels.kv_write(qkv, self.q_width, self.q_width + self.kv_width, k_pool, v_pool,
                             group.slot_mapping, n)
        y = ctx.workspace.get("attn_out", n, self.q_width, ctx.dtype)
        attention_ops.paged_attention(ctx, qkv, y, k_pool, v_pool, group, self.n_head, self.scale, self.window)
        linear_add(ctx, y, self.proj_weight, self.proj_bias, x, n,
                   may_leave_parts=isinstance(h, LazyNorm) and h.x is x)
