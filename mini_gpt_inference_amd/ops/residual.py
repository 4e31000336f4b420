"""The residual stream as a sum that nobody has added up yet.

In a decode step of few rows, the kernels that add to the residual stream (attention with its
output projection, the feed-forward) are split over workgroups along their inner size, and each
workgroup leaves its share as one of several partial sums instead of meeting the others in one
array: x[row] = base[row] + sum_p partials[p, row].  The kernel that reads the residual next adds
them up on its way in and stores the sum, so the chain never grows.  Before the first layer the
"sum" is the token's and the position's table rows, not yet looked up.

`ctx.pending` holds that state for the step's residual stream `x`; None means x is plain.  A part
that cannot read a pending residual calls settle(ctx, x, n_rows) first; the arrangement and the
model do that for parts that do not declare `takes_pending_residual`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import kernels

# most rows of a decode-only step that go through the fused kernels.  A workgroup of the attention
# kernel takes one token of a head, two from where that would be more workgroups than compute units
# and four from where two would, so that a head's weights are read once for them; the 50.9M model's
# step against the kernels that share a matrix among all rows: 222 us against 243 at 40 rows, 242 /
# 264 at 64, 311 / 438 at 96, 330 / 455 at 128 (context 170); 340 / 367 at 64 and 530 / 647 at 128
# (context 740).  Steps of more rows than this are not replayed from graphs either.
FUSED_MAX_ROWS = 128


@dataclass
class PendingSums:
    base: Optional[torch.Tensor]        # float32 [rows, width]: where the rows stand now (x or its twin);
                                        # None: the rows are table rows (tables)
    partials: Optional[torch.Tensor]    # float32 [parts, rows, width], or None
    n_parts: int
    tables: Optional[Tuple] = None      # (token table, position table or None, token ids, positions)


def twin_of(ctx, x: torch.Tensor) -> torch.Tensor:
    """The second array of the residual stream: a kernel that reads rows which other workgroups of
    the same launch still read cannot store their sums in place."""
    return ctx.workspace.get("residual_twin", x.shape[0], x.shape[1], torch.float32)


def plain(x: torch.Tensor) -> PendingSums:
    return PendingSums(x, None, 0)


def take(ctx, x: torch.Tensor) -> Tuple[PendingSums, torch.Tensor]:
    """What a kernel that reads a pending residual needs: (the pending sums, the array it must store
    the settled rows to).  The caller sets ctx.pending to what it leaves behind."""
    pending = ctx.pending if ctx.pending is not None else plain(x)
    on_x = pending.base is not None and pending.base.data_ptr() == x.data_ptr()
    return pending, (twin_of(ctx, x) if on_x else x)


def parts_buffer(ctx, name: str, n_parts: int, n_rows: int, width: int) -> torch.Tensor:
    """Where a kernel leaves its n_parts partial sums [n_parts, n_rows, width].  Every part kind has
    two arrays under its name and takes the one that does not hold the sums still pending: the kernel
    adds those up in its prologue while other workgroups of the same launch already store theirs, so
    two parts of one kind in a row (two attention mixers, two feed-forwards) must not share one."""
    def get(suffix: str) -> torch.Tensor:
        return ctx.workspace.get(name + suffix, n_parts * n_rows, width, torch.float32)[:n_parts * n_rows] \
            .view(n_parts, n_rows, width)
    buf = get("")
    pending = ctx.pending
    if pending is not None and pending.partials is not None \
            and pending.partials.untyped_storage().data_ptr() == buf.untyped_storage().data_ptr():
        buf = get("_second")
    return buf


def settle(ctx, x: torch.Tensor, n_rows: int) -> None:
    """Makes x[:n_rows] plain: adds up what is pending into it."""
    pending = ctx.pending
    if pending is None:
        return
    ctx.pending = None
    if pending.base is None:
        tok, pos, ids, positions = pending.tables
        kernels.embed(ids, positions, tok, pos, x, n_rows)
        return
    if not kernels.residual_settle(pending, x, n_rows):
        raise kernels.KernelError("a residual of this width cannot have been left pending")


def usable(ctx, width: int, n_parts: int = 0) -> bool:
    """Whether this step's residual may be left pending, as n_parts sums: the bfloat16 path, a
    decode-only step of few rows, a width the fused kernels take and no more sums than the next
    reader can add up on its way in."""
    return (ctx.decode_only and not ctx.exact and ctx.dtype == torch.bfloat16 and 0 < ctx.n_rows <= FUSED_MAX_ROWS
            and n_parts <= kernels.fused_parts_limit(width))
