"""The step function: one batch of (request, its next tokens) through the model.

A step is described by flat int32 arrays (one entry per token, per request, per wanted logit
row).  They are written into one pinned host arena, uploaded with one copy into a device arena
of the same layout, and every kernel reads them there; no mask tensor exists, masking is
key position <= query position inside the attention kernels.  The reference builds a
rectangular (B, T) ForwardBatch with a mask instead and never mixes prompts with decoding
(src/minigpt_infer/batch.py:19-65, src/minigpt_infer/engine/engine.py:210-283).
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.kv_store import KVStore
from ..cache.manager import CacheManager
from ..ops import kernels, library
from ..ops.linear import CopyBudget
from ..ops.plan import LaunchPlan
from ..parts.base import GroupView, StepContext, Workspace, WorkspaceFrozen
from ..parts.model import DecoderModel


def _round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


def _bucket(n: int) -> int:
    """Capacities grow in powers of two so that few arenas are ever made."""
    b = 1
    while b < n:
        b *= 2
    return b


def _bucket_tokens(n: int) -> int:
    """The token capacity of a step of n tokens.  A graph made for a capacity runs every kernel over
    all of it, so beyond 64 the capacities lie closer than powers of two: a quarter of the power of
    two below n apart (at most 25 % of padding)."""
    if n <= 64:
        return _bucket(n)
    step = _bucket(n) // 8
    return -(-n // step) * step


class StepArena:
    """Pinned host arrays and their device mirror for steps of up to (n_cap tokens, r_cap requests,
    m_cap logit rows)."""

    def __init__(self, n_cap: int, r_cap: int, m_cap: int, n_groups: int, max_blocks: int,
                 device: torch.device) -> None:
        self.n_cap, self.r_cap, self.m_cap, self.n_groups, self.max_blocks = n_cap, r_cap, m_cap, n_groups, max_blocks
        fields: List[Tuple[str, int, type]] = [
            ("seeds", 2 * m_cap, np.int32),   # 64-bit, first so that it is 8-byte aligned
            ("token_ids", n_cap, np.int32), ("positions", n_cap, np.int32), ("q_req", n_cap, np.int32),
            ("cu_q", r_cap + 1, np.int32), ("seq_lens", r_cap, np.int32), ("state_slots", r_cap, np.int32),
            ("logit_rows", m_cap, np.int32), ("slot_mapping", n_groups * n_cap, np.int32),
            ("block_tables", n_groups * r_cap * max_blocks, np.int32),
            # where the device's history of sampled tokens goes on: every upload sets the device's count
            # (zero unless the caller says otherwise); behind the cache slots and the block tables, so
            # that the three can be uploaded alone (upload_tables)
            ("history_pos", m_cap, np.int32),
            ("temperature", m_cap, np.float32), ("top_k", m_cap, np.int32), ("top_p", m_cap, np.float32),
            ("out_index", m_cap, np.int32),
        ]
        total = sum(_round_up(n, 4) for _, n, _ in fields)
        self.host_t = torch.zeros(total, dtype=torch.int32, pin_memory=device.type == "cuda")
        self.dev_t = torch.zeros(total, dtype=torch.int32, device=device)
        host_np = self.host_t.numpy()
        self.h: Dict[str, np.ndarray] = {}
        self.d: Dict[str, torch.Tensor] = {}
        off = 0
        for name, n, typ in fields:
            self.h[name] = host_np[off:off + n].view(typ)
            dv = self.dev_t[off:off + n]
            self.d[name] = dv.view(torch.float32) if typ is np.float32 else dv
            if name == "slot_mapping":
                self._tables_begin = off
            off += _round_up(n, 4)
            if name == "history_pos":
                self._tables_end = off
        # the addresses of the arrays that the cache manager fills at every step
        self.h_addr: Dict[str, int] = {name: int(self.h[name].ctypes.data) for name in
                                       ("positions", "q_req", "cu_q", "seq_lens", "slot_mapping", "block_tables")}
        self.h["seeds"] = self.h["seeds"].view(np.uint64)
        self.d["seeds"] = self.d["seeds"].view(torch.int64)
        self.tokens_out = torch.zeros(m_cap, dtype=torch.int32, device=device)
        self.tokens_host = torch.zeros(m_cap, dtype=torch.int32, pin_memory=device.type == "cuda")
        self._uploaded: Optional[torch.cuda.Event] = None

    def upload(self) -> None:
        self.dev_t.copy_(self.host_t, non_blocking=True)
        if self.dev_t.is_cuda:
            if self._uploaded is None:
                self._uploaded = torch.cuda.Event()
            self._uploaded.record()

    def upload_tables(self) -> None:
        """Uploads the cache slots of the step's tokens, the block tables and the history count only.
        For steps that go on from what the device itself made of the last ones (tokens, positions,
        lengths): the new pages, the slot of the first new token (the device looked it up before its
        page was in the table) and where the history goes on are all the host has to add."""
        a, b = self._tables_begin, self._tables_end
        self.dev_t[a:b].copy_(self.host_t[a:b], non_blocking=True)
        if self.dev_t.is_cuda:
            if self._uploaded is None:
                self._uploaded = torch.cuda.Event()
            self._uploaded.record()

    def host_ready(self) -> None:
        """Call before writing the host arrays: the copy of the last upload reads them when the
        device gets there, which may be later than the host's next step."""
        if self._uploaded is not None:
            self._uploaded.synchronize()


@dataclass
class StepShape:
    n_tokens: int
    n_req: int
    n_logits: int
    max_q_len: int
    max_seq_len: int
    q_lens: List[int]
    ctx_lens: List[int]
    slots: List[int]
    rows_in_order: bool = False     # the wanted logit rows are 0, 1, ..., n_tokens - 1: every token's, in order


@dataclass
class _StepGraph:
    """A step shape seen before: how often; its launches as a plan (recorded when it first came) and,
    once captured, the graph; each with the arena and the state of the workspace it is bound to."""
    seen: int = 0
    graph: Optional[torch.cuda.CUDAGraph] = None
    arena: Optional[StepArena] = None
    generation: int = -1
    logits: Optional[torch.Tensor] = None
    plan: Optional[LaunchPlan] = None
    plan_arena: Optional[StepArena] = None
    plan_generation: int = -1
    plan_logits: Optional[torch.Tensor] = None


class ModelRunner:
    """Owns the device side of stepping: arenas, workspace, the cache's pools, the model.

    A step's first coming runs the model's Python, one launch per kernel (about 10 us of host time
    each), and for a model whose parts all allow it (Part.graph_safe) records the launches; the
    second coming of the shape makes them from C++ (ops.plan.LaunchPlan), the third captures them in
    a HIP graph that every later one replays, since the host's launches, not the kernels, bound a
    step of a few hundred tokens.  A shape is the tuple of the requests' token counts and the number
    of logit rows; everything else a kernel reads comes from the arena's device arrays."""

    MAX_STEP_GRAPHS = 64
    CAPTURE_AT = 3     # a shape is captured when it comes for the third time (capturing costs a step's launches again)

    def __init__(self, model: DecoderModel, cache: CacheManager, store: KVStore, dtype: torch.dtype,
                 device: torch.device, max_positions: Optional[int], graph_steps: bool = True,
                 derived_weight_bytes: Optional[int] = None) -> None:
        self.model, self.cache, self.store = model, cache, store
        self.copy_budget = CopyBudget(derived_weight_bytes)     # what copies of matrices made at first use may take
        self.dtype, self.device = dtype, device
        self.exact = dtype == torch.float32
        self.max_positions = max_positions
        self.vocab_size = model.spec.vocab_size
        self.workspace = Workspace(device)
        self.graph_steps = graph_steps and device.type == "cuda" and model.graph_safe
        self.plan_steps = device.type == "cuda" and model.plan_safe      # launches recorded and made again from C++
        self.num_planned_steps = 0        # steps whose launches came from a recorded plan
        # a check for tests and for whoever writes a part: a step whose shape has a plan runs through the
        # model's Python again and its launches are compared with the plan's (environment MGPT_VERIFY_PLANS=1)
        self.verify_plans = os.environ.get("MGPT_VERIFY_PLANS", "") not in ("", "0")
        self._step_graphs: Dict[Tuple, _StepGraph] = {}     # by exact shape, least recently used first; at most MAX_STEP_GRAPHS
        self._bucket_graphs: Dict[Tuple, _StepGraph] = {}   # by capacities: as many as there are buckets
        self.num_replayed_steps = 0
        self.num_graph_captures = 0       # HIP graphs recorded so far, decode steps' and other steps'
        self._arenas: Dict[Tuple[int, int, int], StepArena] = {}
        self.n_groups = len(cache.groups)
        self.page_sizes = torch.tensor([g.page_size for g in cache.groups], dtype=torch.int32, device=device)
        # enough block-table columns for the longest sequence this model can hold
        if max_positions is not None:
            self.max_blocks = max(1, max(-(-max_positions // g.page_size) for g in cache.groups))
        else:
            self.max_blocks = max(g.num_pages for g in cache.groups)

    # ------------------------------------------------------------------ arenas
    def arena(self, n_tokens: int, n_req: int, n_logits: int) -> StepArena:
        key = (_bucket_tokens(max(n_tokens, 1)), _bucket(max(n_req, 1)), _bucket(max(n_logits, 1)))
        a = self._arenas.get(key)
        if a is None:
            a = StepArena(*key, self.n_groups, self.max_blocks, self.device)
            self._arenas[key] = a
        return a

    # ------------------------------------------------------------------ describing a step
    def describe(self, arena: StepArena, slots: Sequence[int], ctx_lens: Sequence[int], q_lens: Sequence[int],
                 tokens: Sequence[int], logit_rows: Sequence[int]) -> StepShape:
        """Fills the arena for requests given by their cache slots: request i brings q_lens[i] tokens
        (its part of the flat `tokens`) on top of ctx_lens[i] cached ones.  logit_rows index `tokens`."""
        arena.host_ready()
        h, a = arena.h, arena.h_addr
        max_seq = self.check_positions(ctx_lens, q_lens)
        n = self.cache.build_step(slots, ctx_lens, q_lens, arena.n_cap, arena.r_cap, arena.max_blocks,
                                  a["positions"], a["q_req"], a["cu_q"], a["seq_lens"], a["slot_mapping"],
                                  a["block_tables"])
        if n != len(tokens):
            raise ValueError(f"the step's requests bring {n} tokens, but {len(tokens)} token ids were given")
        ids = h["token_ids"]
        ids[:n] = tokens          # a list or an array
        ids[n:] = 0
        # one comparison for both ends: a negative id is a huge unsigned one
        if n and int(ids[:n].view(np.uint32).max()) >= self.vocab_size:
            raise ValueError(f"token id outside 0..{self.vocab_size - 1}")
        r, m = len(slots), len(logit_rows)
        h["state_slots"][:r] = slots
        h["state_slots"][r:] = -1
        rows = np.asarray(logit_rows, dtype=np.int32)
        if m and (rows.min() < 0 or rows.max() >= n):
            raise ValueError("a wanted logit row lies outside the step's tokens")
        h["logit_rows"][:m] = rows
        h["logit_rows"][m:] = 0
        q_lens = list(q_lens)
        return StepShape(n, r, m, max(q_lens, default=0), max_seq, q_lens, list(ctx_lens), list(slots),
                         rows_in_order=self._rows_in_order(arena, n, m))

    @staticmethod
    def _rows_in_order(arena: StepArena, n: int, m: int) -> bool:
        return m == n and bool((arena.h["logit_rows"][:m] == np.arange(m, dtype=np.int32)).all())

    def check_positions(self, ctx_lens: Sequence[int], q_lens: Sequence[int]) -> int:
        """The longest sequence after the step; refuses positions the model does not have
        (reference: src/minigpt_infer/model.py:177-182)."""
        max_seq = max((c + q for c, q in zip(ctx_lens, q_lens)), default=0)
        if self.max_positions is not None and max_seq > self.max_positions:
            raise ValueError(f"position {max_seq - 1} >= block_size={self.max_positions}: "
                             "the position table has no such row")
        return max_seq

    def shape_of(self, arena: StepArena, n: int, r: int, m: int, q_lens: List[int], ctx_lens: List[int],
                 slots: List[int]) -> StepShape:
        h = arena.h
        ids = h["token_ids"][:n]
        if n and (ids.min() < 0 or ids.max() >= self.vocab_size):
            raise ValueError(f"token id outside 0..{self.vocab_size - 1}")
        max_seq = self.check_positions(ctx_lens, q_lens)
        return StepShape(n, r, m, max(q_lens, default=0), max_seq, q_lens, ctx_lens, slots,
                         rows_in_order=self._rows_in_order(arena, n, m))

    # ------------------------------------------------------------------ running
    def context(self, arena: StepArena, shape: StepShape, padded: bool, workspace: Optional[Workspace] = None,
                lead_cap: Optional[int] = None) -> StepContext:
        """What the parts see of the step.  padded: every kernel runs over the arena's capacities (rows,
        requests, logit rows) instead of the step's own counts.  lead_cap (with padded): the context
        of a bucket of steps with prompt portions, in which nothing may depend on the step at hand
        but the capacities and lead_cap."""
        d = arena.d
        groups = []
        for g, geo in enumerate(self.cache.groups):
            groups.append(GroupView(
                page_size=geo.page_size, window=geo.window,
                slot_mapping=d["slot_mapping"][g * arena.n_cap:(g + 1) * arena.n_cap],
                block_tables=d["block_tables"][g * arena.r_cap * arena.max_blocks:
                                               (g + 1) * arena.r_cap * arena.max_blocks]
                .view(arena.r_cap, arena.max_blocks),
                k_pools=self.store.k_pools(g), v_pools=self.store.v_pools(g)))
        bucket = padded and lead_cap is not None
        return StepContext(
            n_tokens=shape.n_tokens, n_rows=arena.n_cap if padded else shape.n_tokens,
            n_req=shape.n_req, n_logits=shape.n_logits, m_rows=arena.m_cap if padded else shape.n_logits,
            token_ids=d["token_ids"], positions=d["positions"], q_req=d["q_req"], cu_q=d["cu_q"],
            seq_lens=d["seq_lens"], state_slots=d["state_slots"], logit_rows=d["logit_rows"],
            groups=groups, state_pools=self.store.state_pools, dtype=self.dtype,
            workspace=workspace or self.workspace,
            max_q_len=arena.n_cap if bucket else shape.max_q_len, max_seq_len=shape.max_seq_len,
            decode_only=False if bucket else shape.max_q_len <= 1,
            host_q_lens=None if bucket else shape.q_lens, host_ctx_lens=None if bucket else shape.ctx_lens,
            host_state_slots=None if bucket else shape.slots, exact=self.exact, padded=padded,
            lead_cap=lead_cap or 0, copy_budget=self.copy_budget, logit_rows_in_order=shape.rows_in_order)

    def run(self, arena: StepArena, shape: StepShape) -> torch.Tensor:
        """Uploads the arena and runs the model.  Returns float32 logits [n_logits, vocab] (in the
        workspace: the next step overwrites them).

        Two kinds of graphs, both made when what they stand for has come CAPTURE_AT times: one for an
        exact shape (the requests' token counts and the number of logit rows), which runs only the
        step's own rows; and one for a bucket (the arena's capacities and how many tokens the leading
        single-token requests may take), padded to those, which serves every step of the bucket
        whatever its requests bring."""
        arena.upload()
        if not self.plan_steps and not self.graph_steps:
            with kernels.pinned_stream():
                return self.model.forward(self.context(arena, shape, padded=False))
        exact = self._entry((tuple(shape.q_lens), shape.n_logits, shape.rows_in_order))
        if not self.graph_steps:
            return self._planned_or_recorded(exact, arena, shape)
        if self._live(exact, arena):
            exact.graph.replay()
            self.num_replayed_steps += 1
            return exact.logits
        lead = 0
        while lead < shape.n_req and shape.q_lens[lead] == 1:
            lead += 1
        lead_cap = min(-(-lead // 16) * 16, arena.n_cap)
        bucket = self._bucket_graphs.setdefault((arena.n_cap, arena.r_cap, arena.m_cap, lead_cap), _StepGraph())
        exact.seen += 1
        bucket.seen += 1
        if exact.seen < self.CAPTURE_AT and self._live(bucket, arena):
            bucket.graph.replay()
            self.num_replayed_steps += 1
            return bucket.logits[:shape.n_logits]
        logits = self._planned_or_recorded(exact, arena, shape)
        if exact.seen >= self.CAPTURE_AT:
            self._capture(exact, arena, shape, None)
        elif bucket.seen >= self.CAPTURE_AT and not self._live(bucket, arena):
            self._capture(bucket, arena, shape, lead_cap)
        return logits

    def _plan_live(self, entry: _StepGraph, arena: StepArena) -> bool:
        return (entry.plan is not None and entry.plan_arena is arena
                and entry.plan_generation == self.workspace.generation)

    def _planned_or_recorded(self, entry: _StepGraph, arena: StepArena, shape: StepShape) -> torch.Tensor:
        """The step's own rows, eagerly: from the shape's recorded plan if it has a valid one, else
        through the model's Python, which records the plan."""
        with kernels.pinned_stream():
            if not self.plan_steps:
                return self.model.forward(self.context(arena, shape, padded=False))
            if self._plan_live(entry, arena):
                if self.verify_plans:
                    # the step through the model's Python once more, which must make the plan's launches
                    with library.record() as launches:
                        self.model.forward(self.context(arena, shape, padded=False))
                    diff = entry.plan.difference(launches)
                    if diff is not None:
                        raise RuntimeError("a part that promises plan_safe launched otherwise for a step of the "
                                           "same shape: " + diff)
                else:
                    entry.plan.run()
                self.num_planned_steps += 1
                return entry.plan_logits
            with library.record() as launches:
                logits = self.model.forward(self.context(arena, shape, padded=False))
        entry.plan, entry.plan_arena = LaunchPlan(launches), arena
        entry.plan_generation, entry.plan_logits = self.workspace.generation, logits
        return logits

    def _entry(self, key: Tuple) -> _StepGraph:
        entry = self._step_graphs.pop(key, None)
        if entry is None:
            while len(self._step_graphs) >= self.MAX_STEP_GRAPHS:
                # the shape that has not come for the longest time goes, the others keep their graphs
                del self._step_graphs[next(iter(self._step_graphs))]
            entry = _StepGraph()
        self._step_graphs[key] = entry      # the dict keeps insertion order: the newest use is last
        return entry

    def _live(self, entry: _StepGraph, arena: StepArena) -> bool:
        return (entry.graph is not None and entry.arena is arena
                and entry.generation == self.workspace.generation)

    def _capture(self, entry: _StepGraph, arena: StepArena, shape: StepShape, lead_cap: Optional[int]) -> None:
        """Records the step that the arena holds for the next of its shape (lead_cap None) or of its
        bucket.  A bucket's graph runs over more rows than the eager step before it did, so it runs
        once eagerly first: every buffer it needs exists then."""
        def forward():
            with kernels.pinned_stream():
                if lead_cap is None and self._plan_live(entry, arena):
                    entry.plan.run()       # the same launches, without the model's Python
                    return entry.plan_logits
                ctx = self.context(arena, shape, padded=lead_cap is not None, lead_cap=lead_cap)
                return self.model.forward(ctx)
        entry.graph = None
        self.num_graph_captures += 1
        if lead_cap is not None:
            forward()
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        self.workspace.frozen = True
        try:
            with torch.cuda.stream(side):
                graph.capture_begin()
                try:
                    logits = forward()
                except BaseException:
                    # never leave the stream capturing (the graph object's destructor synchronizes
                    # the device); the capture is lost, so what ending it reports is of no interest
                    try:
                        graph.capture_end()
                    except RuntimeError:
                        pass
                    raise
                graph.capture_end()
        except WorkspaceFrozen:
            return   # a buffer would have had to grow: this shape stays eager
        finally:
            self.workspace.frozen = False
            torch.cuda.current_stream().wait_stream(side)
        entry.graph, entry.arena, entry.generation, entry.logits = graph, arena, self.workspace.generation, logits

    def step(self, slots: Sequence[int], ctx_lens: Sequence[int], q_lens: Sequence[int], tokens: Sequence[int],
             logit_rows: Sequence[int]) -> torch.Tensor:
        """The step function for callers that hold cache slots themselves (trace replay, tests)."""
        arena = self.arena(len(tokens), len(slots), len(logit_rows))
        shape = self.describe(arena, slots, ctx_lens, q_lens, tokens, logit_rows)
        return self.run(arena, shape)
