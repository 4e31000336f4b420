"""Feed-forward parts.  A feed-forward adds its output into the residual stream."""

from __future__ import annotations

from typing import Dict

import torch

from ..ops import kernels
from ..ops.linear import linear
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

    def forward_add(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        n = ctx.n_rows
        u = ctx.workspace.get("ff_hidden", n, self.hidden, ctx.dtype)
        linear(ctx, h, self.fc_weight, self.fc_bias, u, n, _ACTIVATIONS[self.activation])
        linear(ctx, u, self.proj_weight, self.proj_bias, x, n, kernels.EPI_RESIDUAL)
