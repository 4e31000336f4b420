"""Arrangements: how a layer's norm, mixer and feed-forward sit around the residual stream."""

from __future__ import annotations

from typing import Mapping, Optional, Tuple

import torch

from ..ops import residual
from ..ops.linear import LazyNorm
from .base import CacheBinding, Part, StepContext, register_arrangement
from .feedforward import FeedForward
from .mixers import Mixer
from .positions import PositionEncoding


class Arrangement(Part):
    """How a layer's parts sit around the residual stream.  `roles` names the parts it arranges (the
    model refuses a layer whose parts are others); run() gets them by role, and for every mixer role
    the binding of this run's cache."""

    category = "arrangement"
    roles: Optional[Tuple[str, ...]] = None     # None: whatever the layer brings

    def run(self, ctx: StepContext, x: torch.Tensor, parts: Mapping[str, Part],
            bindings: Mapping[str, CacheBinding], position: PositionEncoding) -> None:
        raise NotImplementedError


@register_arrangement("pre_norm")
class PreNorm(Arrangement):
    """x = x + mixer(norm1(x)); x = x + ff(norm2(x)) (reference: src/minigpt_infer/model.py:112-115)."""

    graph_safe = True

    plan_safe = True
    takes_pending_residual = True
    roles = ("norm1", "mixer", "norm2", "feed_forward")

    def __init__(self, width: int) -> None:
        self.width = int(width)

    def run(self, ctx, x, parts, bindings, position) -> None:
        norm1, mixer, norm2, feed_forward = (parts[r] for r in self.roles)
        binding = bindings["mixer"]
        # the norms are handed on uncomputed: a linear layer that can normalise in its prologue
        # does, everything else calls .tensor(ctx) and gets the normed rows.  A part that does not
        # know of a residual whose sums are still pending gets a plain one.
        n = ctx.n_rows
        if not mixer.takes_pending_residual:
            residual.settle(ctx, x, n)
        mixer.forward_add(ctx, LazyNorm(norm1, x, n), x, binding, position)
        if not feed_forward.takes_pending_residual:
            residual.settle(ctx, x, n)
        feed_forward.forward_add(ctx, LazyNorm(norm2, x, n), x)
