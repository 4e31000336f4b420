"""Feed-forward parts.  A feed-forward adds its output into the residual stream."""

from __future__ import annotations

from typing import Dict

import torch

from ..ops import kernels, residual
from ..ops.linear import LazyNorm, linear, linear_add, packed_weight, plain_residual
from .base import MATRIX, Part, StepContext, VECTOR, WeightRequest, register_feed_forward

_ACTIVATIONS = {"gelu_tanh": kernels.EPI_GELU}


class FeedForward(Part):
    category = "feed_forward"

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        """x[:n_rows] += ff(h[:n_rows]); h is a tensor or an ops.linear.LazyNorm (see Mixer.forward_add)."""
        raise NotImplementedError


@register_feed_forward("dense_mlp")
class DenseMLP(FeedForward):
    """u = h Wfc^T (+ b); g = 0.5 u (1 + tanh(sqrt(2/pi)(u + 0.044715 u^3))); m = g Wproj^T (+ b)
    (reference: src/minigpt_infer/model.py:96-101; there the hidden size is 4*n_embd, here it is
    a parameter)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True

    def __init__(self, width: int, hidden: int, bias: bool, activation: str = "gelu_tanh") -> None:
        if activation not in _ACTIVATIONS:
            raise ValueError(f"activation {activation!r} has no kernel epilogue; known: {sorted(_ACTIVATIONS)}")
        self.width, self.hidden, self.has_bias = int(width), int(hidden), bool(bias)
        self.activation = activation
        self.fc_weight = self.fc_bias = self.proj_weight = self.proj_bias = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = {"fc_weight": WeightRequest((self.hidden, self.width), MATRIX),
               "proj_weight": WeightRequest((self.width, self.hidden), MATRIX)}
        if self.has_bias:
            req["fc_bias"] = WeightRequest((self.hidden,), VECTOR)
            req["proj_bias"] = WeightRequest((self.width,), VECTOR)
        return req

    def _forward_add_fused(self, ctx: StepContext, h, x: torch.Tensor) -> bool:
        """A decode-only step of few rows: one kernel from the residual (a sum, as the kernels
        before left it) through LayerNorm, both products and the activation to this part's addition
        to the residual, left as one partial sum per 64 hidden units.  False, with nothing launched,
        where that kernel does not apply."""
        parts_n = kernels.fused_mlp_parts(self.hidden)
        if not (isinstance(h, LazyNorm) and h._tensor is None and h.rows is None and h.x is x
                and getattr(h.norm, "fusable_layer_norm", False) and parts_n and residual.usable(ctx, self.width, parts_n)
                and self.activation == "gelu_tanh" and self.fc_weight.dtype == torch.bfloat16
                and self.proj_weight.dtype == torch.bfloat16):
            return False
        wfc, wproj = packed_weight(self.fc_weight, ctx), packed_weight(self.proj_weight, ctx)
        if wfc is None or wproj is None:
            return False
        n = ctx.n_rows
        if ctx.pending is not None and ctx.pending.base is None:
            residual.settle(ctx, x, n)      # table rows: this kernel reads residual rows only
        pending, settled = residual.take(ctx, x)
        parts = residual.parts_buffer(ctx, "feed_forward_parts", parts_n, n, self.width)
        if not kernels.fused_mlp_decode(pending, settled, h.norm.weight, h.norm.bias, h.norm.eps, wfc, self.fc_bias,
                                        wproj, self.proj_bias, parts, n, self.hidden):
            return False
        ctx.pending = residual.PendingSums(settled, parts, parts_n)
        return True

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        if self._forward_add_fused(ctx, h, x):
            return
        plain_residual(ctx, h, x)
        n = ctx.n_rows
        u = ctx.workspace.get("ff_hidden", n, self.hidden, ctx.dtype)
        linear(ctx, h, self.fc_weight, self.fc_bias, u, n, _ACTIVATIONS[self.activation])
        # (a caller that hands over a LazyNorm of x itself knows that x may be left as a sum)
        linear_add(ctx, u, self.proj_weight, self.proj_bias, x, n,
                   may_leave_parts=isinstance(h, LazyNorm) and h.x is x)
