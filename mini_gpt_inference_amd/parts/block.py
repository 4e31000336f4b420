"""Arrangements: how a layer's norm, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

import torch

from .base import CacheBinding, Part, StepContext, register_arrangement
from .feedforward import FeedForward
from .mixers import Mixer
from .positions import PositionEncoding


class Arrangement(Part):
    category = "arrangement"

    def run(self, ctx: StepContext, x: torch.Tensor, norm1: Part, mixer: Mixer, norm2: Part,
            feed_forward: FeedForward, binding: CacheBinding, position: PositionEncoding) -> None:
        raise NotImplementedError


@register_arrangement("pre_norm")
class PreNorm(Arrangement):
    """x = x + mixer(norm1(x)); x = x + ff(norm2(x)) (reference: src/minigpt_infer/model.py:112-115)."""

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, norm1, mixer, norm2, feed_forward, binding, position) -> None:
        n = ctx.n_rows
        h = ctx.workspace.get("normed", n, self.width, ctx.dtype)
        norm1.forward(ctx, x, h, n)
        mixer.forward_add(ctx, h, x, binding, position)
        norm2.forward(ctx, x, h, n)
        feed_forward.forward_add(ctx, h, x)
