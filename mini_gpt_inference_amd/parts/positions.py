"""Position encodings.

A position encoding can act in two places: on the residual stream right after the
token embedding (`embedding_table`), or on queries and keys inside a mixer
(`rotate`).  A part implements the hooks it needs and leaves the others alone.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Part, StepContext, TABLE, WeightRequest, register_position


class PositionEncoding(Part):
    category = "position"
    max_positions: Optional[int] = None   # hard bound on positions, None = unbounded
    rotates = False                       # True if rotate() changes queries and keys

    def embedding_table(self) -> Optional[torch.Tensor]:
        """A [max_positions, width] table whose row pos[t] is added to token t's embedding."""
        return None

    def rotate(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor, n_tokens: int) -> None:
        """Acts on projected queries and keys in place, before the keys are cached."""
        return None


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """x0[t] += pos_emb[pos_t] with pos_t the absolute position, which must be < max_positions
    (reference: src/minigpt_infer/model.py:124,177-183)."""

    graph_safe = True

    plan_safe = True

    def __init__(self, max_positions: int, width: int) -> None:
        self.max_positions, self.width = int(max_positions), int(width)
        self.weight: Optional[torch.Tensor] = None

    def weight_requests(self) -> Dict[str, WeightRequest]:
        return {"weight": WeightRequest((self.max_positions, self.width), TABLE)}

    def embedding_table(self) -> Optional[torch.Tensor]:
        return self.weight


@register_position("none")
class NoPositions(PositionEncoding):
    """No position signal at all."""

    graph_safe = True

    plan_safe = True

    def __init__(self) -> None:
        pass
