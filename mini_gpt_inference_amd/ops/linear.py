"""Chooses the matrix-product kernel for a linear layer, and carries a LayerNorm that has not
been computed yet to the kernel that can compute it in its prologue."""

from __future__ import annotations

from typing import Optional, Union

import torch

from . import kernels, residual


class LazyNorm:
    """The normed residual stream, not yet computed: norm(x[rows]) (or norm(x)).  A linear layer
    that reads it may compute the norm in its own prologue; anyone else calls tensor()."""

    def __init__(self, norm, x: torch.Tensor, n_rows: int, rows: Optional[torch.Tensor] = None,
                 buffer: str = "normed") -> None:
        self.norm, self.x, self.n_rows, self.rows, self.buffer = norm, x, n_rows, rows, buffer
        self._tensor: Optional[torch.Tensor] = None

    def tensor(self, ctx) -> torch.Tensor:
        if self._tensor is None:
            h = ctx.workspace.get(self.buffer, self.n_rows, self.x.shape[1], ctx.dtype)
            pending = getattr(ctx, "pending", None)
            if pending is not None:
                # the residual is still a sum: a LayerNorm adds it up on its way in (and, where it
                # goes over all the step's rows, stores the sums: the residual is plain again),
                # anything else needs plain rows first
                norm = self.norm
                all_rows = self.rows is None and self.n_rows >= ctx.n_rows
                if (getattr(norm, "fusable_layer_norm", False)
                        and kernels.residual_layer_norm(pending, norm.weight, norm.bias, norm.eps, self.rows, h,
                                                        self.n_rows, settled=self.x if all_rows else None)):
                    if all_rows:
                        ctx.pending = None
                else:
                    residual.settle(ctx, self.x, ctx.n_rows)
                    pending = None
            if pending is None:
                self.norm.forward(ctx, self.x, h, self.n_rows, rows=self.rows)
            self._tensor = h
        return self._tensor


# Derived copies of a matrix (folded with a LayerNorm, packed for the decode kernel) hang on the
# matrix tensor itself, so they live exactly as long as it does.
_DERIVED = "_mgpt_derived"


def _derived(w: torch.Tensor) -> dict:
    """The table of w's derived copies.  It hangs on the tensor that owns the memory (a view made
    afresh at every call would take its table with it when it goes), one table per place and shape."""
    owner = w._base if w._base is not None else w
    tables = getattr(owner, _DERIVED, None)
    if tables is None:
        tables = {}
        setattr(owner, _DERIVED, tables)
    return tables.setdefault((w.data_ptr(), tuple(w.shape), tuple(w.stride())), {})


def derived_bytes(w: torch.Tensor) -> int:
    """Bytes of device memory that the derived copies of w hold (folded with a LayerNorm, packed
    for the decode kernels), counting every copy of every view of w's storage once."""
    owner = w._base if w._base is not None else w
    seen, total = set(), 0

    def walk(obj) -> None:
        nonlocal total
        if isinstance(obj, torch.Tensor):
            if obj.data_ptr() not in seen:
                seen.add(obj.data_ptr())
                total += obj.numel() * obj.element_size()
        elif isinstance(obj, (tuple, list)):
            for item in obj:
                walk(item)
        elif isinstance(obj, dict):
            for item in obj.values():
                walk(item)

    walk(getattr(owner, _DERIVED, None))
    return total


class CopyBudget:
    """Device memory that derived copies of matrices may still take (EngineConfig.derived_weight_bytes).
    A copy that does not fit is not made: its matrix is then read as it was loaded (row-major through
    the decode kernels, its LayerNorm by the LayerNorm kernel), slower and with the same results up
    to rounding."""

    def __init__(self, limit: Optional[int]) -> None:
        self.limit = limit          # None: no bound
        self.used = 0

    def take(self, n_bytes: int) -> bool:
        if self.limit is not None and self.used + n_bytes > self.limit:
            return False
        self.used += n_bytes
        return True


def _budget(ctx) -> Optional[CopyBudget]:
    return getattr(ctx, "copy_budget", None) if ctx is not None else None


def folded_layer_norm(norm, w: torch.Tensor, bias: Optional[torch.Tensor], ctx=None):
    """(folded matrix, column sums, folded bias): the matrix with the LayerNorm's gain and bias
    folded in, made once per (norm, matrix, bias).  None if the step's budget for copies has no
    room for it."""
    key = ("folded", norm.weight.data_ptr(), 0 if norm.bias is None else norm.bias.data_ptr(),
           0 if bias is None else bias.data_ptr())
    d = _derived(w)
    hit = d.get(key)
    if hit is None:
        budget = _budget(ctx)
        if budget is not None and not budget.take(w.numel() * w.element_size() + 8 * w.shape[0]):
            return None
        hit = d[key] = kernels.fold_layer_norm(w, norm.weight, norm.bias, bias)
    return hit


def packed_weight(w: torch.Tensor, ctx=None) -> Optional[torch.Tensor]:
    """The matrix in the layout the decode kernel reads fastest, made once per matrix (at its first
    decode step, before any graph is captured).  None if the kernel's layout does not take the
    shape, or if the step's budget for copies has no room for it."""
    d = _derived(w)
    if "packed" not in d:
        budget = _budget(ctx)
        if budget is not None and w.shape[1] % 32 == 0 \
                and not budget.take(-(-w.shape[0] // 16) * 16 * w.shape[1] * w.element_size()):
            return None         # (not remembered: a later step never has more room, but a test may lift the bound)
        d["packed"] = kernels.pack_weight(w)
    return d["packed"]


# A LayerNorm is folded into the product that reads it only for outputs this wide at most, and for
# this many rows unless the decode kernel deals the rows out in groups of 16: every workgroup
# converts the float32 residual rows it multiplies, which beyond these costs more than a LayerNorm
# kernel of its own (at 64 rows in one workgroup the decode step of the 50.9M model took 0.397 ms
# with the fold and 0.375 ms without).
FOLD_MAX_ROWS = 32
FOLD_MAX_OUT = 4096
# ... except at few rows, where the LayerNorm kernel's own launch costs more than the conversion
# (the GPT-2-XL shape, outputs of 4800 and 6400: 957 us a step of 24 layers against 1062 at one
# row, 1361 against 1399 at 16 rows, 1923 against 1741 at 32), but not under an output as wide as a
# vocabulary: every one of its thousands of workgroups would norm the rows again ([50257 x 1600] at
# one row: 43.5 us with the fold, 30.0 without, and the LayerNorm kernel takes 3)
FOLD_ANY_OUT_MAX_ROWS = 16
FOLD_ANY_OUT_MAX_OUT = 8192
# A very wide output (the head, 8192 columns and more) goes to the decode kernel while rows x inner
# size stays within this, and to the tiled kernel beyond: that one streams the matrix at nearly the
# same rate whatever the rows (50304 x 512: 10.2 us at 1 row, 11.4 at 32, 14.0 at 64), the decode
# kernel is ahead by up to a microsecond at few rows and a short inner size and slows down with every
# row (9.4, 16.4, 28.5 us; at an inner size of 1600 it is behind from 4 rows on).
WIDE_OUT = 8192
WIDE_OUT_DECODE_WORK = 8192
# The decode kernel's time grows with the rows (every workgroup loads all of them for its 16 output
# columns), the tiled kernel's hardly: under a large matrix with a wide output the tiled kernel (32 x
# 32 tiles, several steps on their way from memory) is ahead from 17 rows on.  Matrices from memory,
# decode kernel against tiled: [4800 x 1600] 8.5 / 8.5 us at 16 rows, 10.6 / 8.5 at 24, 11.7 / 8.5 at
# 32, 18.8 / 10.0 at 64; [6400 x 1600] 9.3 / 9.1, 11.4 / 9.3, 12.7 / 9.3, 19.8 / 12.0; under smaller
# matrices the decode kernel stays ahead up to 64 rows ([3072 x 768] 5.0 / 5.6 at 32, 6.2 / 5.6 at
# 64; [1600 x 1600] 5.8 / 8.4 and 8.0 / 8.4).  A long inner size under a narrow output is split over
# workgroups by either; there the tiled kernel with its joining kernel is ahead from 33 rows on
# ([1600 x 6400]: the decode kernel's first half alone, its sums left pending, 20.0 us at 64 rows, the
# tiled pair 15.1; at 32 rows about 11.5 against 12.7).
TILED_FROM_ROWS = 17
TILED_MIN_OUT = 4096
TILED_MIN_MATRIX = 6_000_000
TILED_ANY_OUT_FROM_ROWS = 33


def tiled_at_few_rows(n_rows: int, w: torch.Tensor) -> bool:
    """Whether a product of few rows (the decode kernel takes up to 64; linear_add asks for up to
    LEAVE_PARTS_MAX_ROWS) goes to the tiled kernel rather than the decode kernel."""
    if w.shape[0] * w.shape[1] < TILED_MIN_MATRIX:
        return False
    return n_rows >= TILED_ANY_OUT_FROM_ROWS or (n_rows >= TILED_FROM_ROWS and w.shape[0] >= TILED_MIN_OUT)


def as_tensor(ctx, a: Union[torch.Tensor, LazyNorm]) -> torch.Tensor:
    return a.tensor(ctx) if isinstance(a, LazyNorm) else a


class TileBest:
    """Asks a product for the best column of every tile of 16 beside its float32 output: the largest
    value among the columns below `limit` and its column.  The product that can, fills values and
    columns ([rows, out / 16], from the workspace) and sets `filled`."""

    def __init__(self, limit: int) -> None:
        self.limit = int(limit)
        self.values: Optional[torch.Tensor] = None
        self.columns: Optional[torch.Tensor] = None
        self.filled = False


# A split product's parts are left pending for rows this wide, or this many: the LayerNorm kernel
# that then adds them up is one workgroup per row, and for one narrow row costs more than the
# kernel that adds the parts plus the folded LayerNorm it replaces (decode steps on one box, us:
# width 768: 296 against 284 at one row, 333 against 336 at 8, 365 against 369 at 16; width 1600:
# 1748 against 1768, 2049 against 2102, 2439 against 2554)
LEAVE_PARTS_MIN_WIDTH = 1024
LEAVE_PARTS_MIN_ROWS = 8
LEAVE_PARTS_MAX_ROWS = 256     # (the tiled kernel's split; the decode kernel's ends at its 64 rows)


def plain_residual(ctx, h, x: torch.Tensor) -> None:
    """Makes the residual rows x plain for a part that reads or adds to them with ordinary kernels.
    If they are still a sum and h is the LayerNorm of them that the part is about to read, that
    LayerNorm is computed now: its kernel adds the sum up and stores it on the way."""
    if getattr(ctx, "pending", None) is None:
        return
    if isinstance(h, LazyNorm) and h.x is x and h._tensor is None:
        h.tensor(ctx)
    residual.settle(ctx, x, ctx.n_rows)


def linear_add(ctx, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], x: torch.Tensor, n_rows: int,
               may_leave_parts: bool = False) -> None:
    """x[:n_rows] += a[:n_rows] @ w.T (+ bias), x the float32 residual stream.

    may_leave_parts: the caller and whoever reads x next know of ctx.pending.  Then a product whose
    long inner size is split over workgroups anyway (few rows, few column tiles) leaves the
    workgroups' sums as the parts of a pending residual instead of running a second kernel that adds
    them into x; the LayerNorm that reads x next adds them up (LazyNorm.tensor)."""
    leave = (may_leave_parts and getattr(ctx, "pending", None) is None and not ctx.exact
             and ctx.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dtype == torch.bfloat16
             and 0 < n_rows <= LEAVE_PARTS_MAX_ROWS and n_rows == ctx.n_rows and x.is_contiguous()
             and x.shape[1] == w.shape[0] and w.shape[1] % 16 == 0)
    if leave and tiled_at_few_rows(n_rows, w):
        # the tiled kernel's split: its stretches' sums are the parts (2 to 8 of them)
        need = kernels.linear_mfma_partials(n_rows, w.shape[0], w.shape[1], kernels.EPI_RESIDUAL)
        n_parts = need // (n_rows * w.shape[0])
        if 1 < n_parts <= kernels.residual_parts_limit(w.shape[0]):
            buf = ctx.workspace.get("residual_parts", n_parts * n_rows, w.shape[0], torch.float32)
            parts = buf[:n_parts * n_rows].view(n_parts, n_rows, w.shape[0])
            if kernels.linear_mfma_parts(a, w, bias, parts, n_rows):
                ctx.pending = residual.PendingSums(x, parts, n_parts)
                return
    elif (leave and n_rows <= 64 and (w.shape[0] >= LEAVE_PARTS_MIN_WIDTH or n_rows >= LEAVE_PARTS_MIN_ROWS)
            and kernels.residual_parts_limit(w.shape[0]) >= 4
            and kernels.linear_skinny_partials(n_rows, w.shape[0], w.shape[1], False, kernels.EPI_RESIDUAL)):
        buf = ctx.workspace.get("residual_parts", 4 * n_rows, w.shape[0], torch.float32)
        parts = buf[:4 * n_rows].view(4, n_rows, w.shape[0])
        n_parts = kernels.linear_decode_parts(a, w, bias, parts, n_rows, w_packed=packed_weight(w, ctx))
        if n_parts:
            assert n_parts == 4
            ctx.pending = residual.PendingSums(x, parts, n_parts)
            return
    linear(ctx, a, w, bias, x, n_rows, kernels.EPI_RESIDUAL)


def linear(ctx, a: Union[torch.Tensor, LazyNorm], w: torch.Tensor, bias: Optional[torch.Tensor],
           out: torch.Tensor, n_rows: int, epilogue: int = kernels.EPI_NONE, scatter=None,
           tile_best: Optional[TileBest] = None) -> bool:
    """out[:n_rows] = a[:n_rows] @ w.T (+ bias) with the epilogue.

    On the bfloat16 path up to 64 rows (fewer for a very wide output) go to the decode step's MFMA kernels (reading the residual
    stream through the folded LayerNorm when `a` is a LazyNorm of a fusable norm and the rows are
    few; splitting a long inner size over workgroups when the rows are many) and more rows to the
    tiled MFMA kernel (which also splits a long inner size when its tiles are few); the 32-bit path, and every shape those refuse, go to the 32-bit FMA kernel.  `scatter` = (k_pool, v_pool,
    slot_mapping, q_width, kv_width) asks for the new keys and values to be stored into their
    pages by the same kernel; the return value says whether that was done."""
    if n_rows == 0:
        return scatter is not None
    if isinstance(a, LazyNorm) and getattr(ctx, "pending", None) is not None:
        a = a.tensor(ctx)      # the kernels below read plain residual rows
    # (the MFMA kernels take inner sizes in steps of 16; any other goes to the general kernel)
    fast = w.dtype == torch.bfloat16 and not ctx.exact and ctx.dtype == torch.bfloat16 and w.shape[1] % 16 == 0
    wide_out = w.shape[0] >= WIDE_OUT and n_rows * w.shape[1] > WIDE_OUT_DECODE_WORK
    if (tile_best is not None and fast and n_rows <= 16 and not wide_out and epilogue == kernels.EPI_NONE
            and scatter is None and w.shape[0] % 16 == 0 and w.shape[1] % 32 == 0
            and not kernels.linear_skinny_partials(n_rows, w.shape[0], w.shape[1], False, epilogue)):
        rows = out.shape[0]
        tile_best.values = ctx.workspace.get("tile_best_values", rows, w.shape[0] // 16, torch.float32)
        tile_best.columns = ctx.workspace.get("tile_best_columns", rows, w.shape[0] // 16, torch.int32)
        if kernels.linear_head_best(as_tensor(ctx, a), w, bias, out, n_rows, tile_best.values, tile_best.columns,
                                    tile_best.limit, w_packed=packed_weight(w, ctx)):
            tile_best.filled = True
            return False
    if fast and n_rows <= 64 and not wide_out and not tiled_at_few_rows(n_rows, w):
        epi = kernels.SK_EPI_QKV if scatter is not None else epilogue
        if (isinstance(a, LazyNorm) and getattr(a.norm, "fusable_layer_norm", False) and a._tensor is None
                and (w.shape[0] <= FOLD_MAX_OUT
                     or (n_rows <= FOLD_ANY_OUT_MAX_ROWS and w.shape[0] <= FOLD_ANY_OUT_MAX_OUT))
                and (n_rows <= FOLD_MAX_ROWS or kernels.linear_skinny_row_groups(n_rows, w.shape[0], w.shape[1]))):
            folded = folded_layer_norm(a.norm, w, bias, ctx)
            if folded is not None:
                wf, colsum, bias_f = folded
                if kernels.linear_skinny(None, wf, bias_f, out, n_rows, epi, ln_x=a.x, ln_colsum=colsum,
                                         ln_eps=a.norm.eps, ln_rows=a.rows, scatter=scatter,
                                         w_packed=packed_weight(wf, ctx)):
                    return scatter is not None
        partials = None
        need = kernels.linear_skinny_partials(n_rows, w.shape[0], w.shape[1], False, epi)
        if need:
            partials = ctx.workspace.get("linear_partials", need, 1, torch.float32)
        if kernels.linear_skinny(as_tensor(ctx, a), w, bias, out, n_rows, epi, scatter=scatter, partials=partials,
                                 w_packed=packed_weight(w, ctx)):
            return scatter is not None
    a = as_tensor(ctx, a)
    if fast and scatter is not None and kernels.linear_mfma(a, w, bias, out, n_rows, epilogue, scatter=scatter):
        return True
    if fast:
        need = kernels.linear_mfma_partials(n_rows, w.shape[0], w.shape[1], epilogue)
        partials = ctx.workspace.get("linear_partials", need, 1, torch.float32) if need else None
        if kernels.linear_mfma(a, w, bias, out, n_rows, epilogue, partials=partials):
            return False
    kernels.linear_generic(a, w, bias, out, n_rows, epilogue)
    return False
