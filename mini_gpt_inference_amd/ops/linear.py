"""Chooses the matrix-product kernel for a linear layer."""

from __future__ import annotations

from typing import Optional

import torch

from . import kernels


def linear(ctx, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           n_rows: int, epilogue: int = kernels.EPI_NONE) -> None:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias) with the epilogue.

    bfloat16 activations with a bfloat16 matrix go to the MFMA kernels (skinny for few rows);
    everything else, and every shape those refuse, goes to the 32-bit FMA kernel."""
    if n_rows == 0:
        return
    if a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and not ctx.exact:
        if kernels.linear_bf16(a, w, bias, out, n_rows, epilogue):
            return
    kernels.linear_generic(a, w, bias, out, n_rows, epilogue)
