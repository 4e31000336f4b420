"""Normalisation parts."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels
from .base import Part, StepContext, VECTOR, WeightRequest, register_norm


@register_norm("layer_norm")
class LayerNorm(Part):
    """y = (x - mean) / sqrt(var_biased + eps) * weight (+ bias) over the last dim, statistics in
    float32 (reference: nn.LayerNorm at src/minigpt_infer/model.py:107,109,127; there eps is the
    library default, here it is a parameter)."""

    graph_safe = True

    plan_safe = True

    category = "norm"
    fusable_layer_norm = True   # a linear kernel may fold weight and bias into its matrix and apply mean, rstd itself

    def __init__(self, width: int, eps: float, bias: bool) -> None:
        self.width, self.eps, self.has_bias = int(width), float(eps), bool(bias)
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        req = {"weight": WeightRequest((self.width,), VECTOR)}
        if self.has_bias:
            req["bias"] = WeightRequest((self.width,), VECTOR)
        return req

    def forward(self, ctx: StepContext, x: torch.Tensor, out: torch.Tensor, n_rows: int,
                rows: Optional[torch.Tensor] = None) -> None:
        """out[i] = norm(x[rows[i]]) (or x[i]); x is the float32 residual stream."""
        kernels.layer_norm(x, self.weight, self.bias, out, n_rows, self.eps, rows)
