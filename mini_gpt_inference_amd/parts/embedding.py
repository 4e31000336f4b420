"""Token embedding and the output head."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import kernels, residual
from ..ops.linear import linear
from .base import MATRIX, Part, StepContext, TABLE, WeightRequest, register_embedding, register_head
from .positions import PositionEncoding


@register_embedding("token_embedding")
class TokenEmbedding(Part):
    """x0[t] = tok_emb[id_t] (+ the position encoding's table row), written to the float32
    residual stream (reference: src/minigpt_infer/model.py:123,183)."""

    graph_safe = True

    plan_safe = True

    category = "embedding"

    def __init__(self, vocab_size: int, width: int) -> None:
        self.vocab_size, self.width = int(vocab_size), int(width)
        self.weight: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"weight": WeightRequest((self.vocab_size, self.width), TABLE)}

    def forward(self, ctx: StepContext, position: PositionEncoding, x: torch.Tensor) -> None:
        table = position.embedding_table()
        if (residual.usable(ctx, self.width, 1) and self.weight.dtype == torch.bfloat16
                and (table is None or table.dtype == torch.bfloat16)):
            # a decode-only step of few rows: the rows are looked up by the kernel that reads the
            # residual first (or by ops.residual.settle, for a part that needs plain rows)
            ctx.pending = residual.PendingSums(None, None, 0, (self.weight, table, ctx.token_ids, ctx.positions))
            return
        kernels.embed(ctx.token_ids, ctx.positions, self.weight, table, x, ctx.n_rows)


@register_head("linear_head")
class LinearHead(Part):
    """logits = h W^T, float32 out, no bias (reference: src/minigpt_infer/model.py:128,187).
    With tied = True the matrix is the token embedding's, one buffer seen twice
    (src/minigpt_infer/model.py:129-130)."""

    graph_safe = True

    plan_safe = True

    category = "head"

    def __init__(self, vocab_size: int, width: int, tied: bool) -> None:
        self.vocab_size, self.width, self.tied = int(vocab_size), int(width), bool(tied)
        self.weight: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"weight": WeightRequest((self.vocab_size, self.width), MATRIX)}

    def forward(self, ctx: StepContext, h: torch.Tensor, logits: torch.Tensor, n_rows: int) -> None:
        linear(ctx, h, self.weight, None, logits, n_rows, tile_best=ctx.tile_best)
