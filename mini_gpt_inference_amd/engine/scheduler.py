"""Python face of the C++ scheduler (csrc/host/scheduler.h)."""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

from ..cache.manager import CacheManager
from ..ops import library

WAITING, RUNNING, FINISHED = 0, 1, 2
FINISH_REASONS = {0: None, 1: "eot", 2: "length", 3: "cancelled"}

_ADD_ERRORS = {
    -1: "the prompt is empty",
    -2: "prompt length + max_tokens exceeds the model's positions (block_size)",
    -3: "the request needs more cache pages than the whole pool holds",
    -4: "bad sampling parameters",
}


class SchedulerError(ValueError):
    pass


@dataclass(frozen=True)
class StepEntry:
    request: int    # scheduler's request id
    ctx: int        # tokens already cached
    q_len: int      # tokens fed in this step
    sample: bool    # the step completes the context: one token is sampled


@dataclass(frozen=True)
class RequestInfo:
    status: int
    finish_reason: Optional[str]
    num_computed: int
    prompt_len: int
    output_len: int
    slot: int


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


class Scheduler:
    def __init__(self, cache: CacheManager, max_batch_size: int, max_num_batched_tokens: int,
                 prefill_chunk: int, mixed: bool, max_positions: int, spare_asker: bool = False) -> None:
        self._lib = library.host()
        self.cache = cache
        self.max_batch_size = max_batch_size
        self._h = self._lib.mgpt_sched_create(cache.handle, max_batch_size, max_num_batched_tokens,
                                              prefill_chunk, int(mixed), max_positions, int(spare_asker))
        if not self._h:
            raise SchedulerError(library.host_error())
        self._counts = np.zeros(3, dtype=np.int32)
        cap = max(max_batch_size, 1)
        self._e = [np.zeros(cap, dtype=np.int32) for _ in range(4)]
        self._o = [np.zeros(cap, dtype=np.int32) for _ in range(4)]
        self._ep = [_p(a) for a in self._e]
        self._op = [_p(a) for a in self._o]
        self._cp = _p(self._counts)

    def __del__(self) -> None:
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mgpt_sched_destroy(h)

    def add_request(self, prompt: Sequence[int], max_tokens: int, eot: Optional[int] = None,
                    temperature: float = 1.0, top_k: Optional[int] = None, top_p: Optional[float] = None,
                    seed: Optional[int] = None) -> int:
        arr = np.ascontiguousarray(np.asarray(list(prompt), dtype=np.int32))
        rid = self._lib.mgpt_sched_add(self._h, _p(arr) if arr.size else None, int(arr.size), int(max_tokens),
                                       -1 if eot is None else int(eot), float(temperature),
                                       0 if top_k is None else int(top_k), 1.0 if top_p is None else float(top_p),
                                       ctypes.c_ulonglong((seed or 0) & (2 ** 64 - 1)), int(seed is not None))
        if rid < 0:
            raise SchedulerError(_ADD_ERRORS.get(rid, f"add_request failed ({rid}) {library.host_error()}"))
        return rid

    def has_work(self) -> bool:
        return bool(self._lib.mgpt_sched_has_work(self._h))

    def cancel(self, rid: int) -> bool:
        return bool(self._lib.mgpt_sched_cancel(self._h, rid))

    def schedule(self) -> Tuple[int, int, int]:
        """Plans the next step.  Returns (tokens, entries, entries that sample)."""
        r = self._lib.mgpt_sched_schedule(self._h, self._cp)
        if r < 0:
            raise SchedulerError(library.host_error())
        return int(self._counts[0]), int(self._counts[1]), int(self._counts[2])

    def entries(self) -> List[StepEntry]:
        n = self._lib.mgpt_sched_entries(self._h, *self._ep, self._e[0].size)
        return [StepEntry(int(self._e[0][i]), int(self._e[1][i]), int(self._e[2][i]), bool(self._e[3][i]))
                for i in range(n)]

    def entry_arrays(self) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
        n = self._lib.mgpt_sched_entries(self._h, *self._ep, self._e[0].size)
        return tuple(a[:n] for a in self._e)

    def fill(self, arena, step_offset: int = 0) -> None:
        """Writes the planned step (or step `step_offset` of a planned burst) into a StepArena's
        host arrays."""
        args = getattr(arena, "_fill_args", None)
        if args is None:      # the arena's addresses never change: make the argument list once
            h = arena.h
            args = arena._fill_args = (
                arena.n_cap, arena.r_cap, arena.m_cap, arena.max_blocks,
                _p(h["token_ids"]), _p(h["positions"]), _p(h["q_req"]), _p(h["cu_q"]), _p(h["seq_lens"]),
                _p(h["slot_mapping"]), _p(h["block_tables"]), _p(h["state_slots"]), _p(h["logit_rows"]),
                _p(h["temperature"]), _p(h["top_k"]), _p(h["top_p"]), _p(h["seeds"]), _p(h["out_index"]))
        arena.host_ready()
        rc = self._lib.mgpt_sched_fill(self._h, self.cache.handle, step_offset, *args)
        if rc != 0:
            raise SchedulerError(f"filling the step failed ({rc}) {library.host_error()}")

    def commit(self, tokens: np.ndarray) -> List[Tuple[int, int, bool, Optional[str]]]:
        """Hands in the sampled tokens (entry order).  Returns (request, token, finished, reason)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        n = self._lib.mgpt_sched_commit(self._h, _p(tokens) if tokens.size else None, int(tokens.size),
                                        *self._op, self._o[0].size)
        if n < 0:
            raise SchedulerError(f"commit failed ({n}) {library.host_error()}")
        ids, toks, fin, why = self._o
        return [(int(ids[i]), int(toks[i]), bool(fin[i]), FINISH_REASONS[int(why[i])]) for i in range(n)]

    def plan_burst(self, max_k: int) -> int:
        """Plans up to max_k decode steps at once (see csrc/host/scheduler.h).  Returns k >= 2, or 0."""
        k = self._lib.mgpt_sched_plan_burst(self._h, int(max_k))
        if k < 0:
            raise SchedulerError(library.host_error())
        return k

    def commit_burst(self, tokens: np.ndarray, k: int, last: bool = True) -> List[Tuple[int, int, bool, Optional[str]]]:
        """tokens[j, i]: what entry i sampled in step j of the burst.  A burst may be handed in in
        several stretches of steps, in order; `last` says that this one ends it."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        cap = tokens.size
        out = [np.zeros(max(cap, 1), dtype=np.int32) for _ in range(4)]
        n = self._lib.mgpt_sched_commit_burst(self._h, _p(tokens), int(k), 1 if last else 0, *[_p(a) for a in out], cap)
        if n < 0:
            raise SchedulerError(f"commit_burst failed ({n}) {library.host_error()}")
        ids, toks, fin, why = out
        return [(int(ids[i]), int(toks[i]), bool(fin[i]), FINISH_REASONS[int(why[i])]) for i in range(n)]

    # -------------------------------------------------------------- inspection
    def _counter(self, which: int) -> int:
        return int(self._lib.mgpt_sched_counter(self._h, which))

    num_preemptions = property(lambda self: self._counter(0))
    num_steps = property(lambda self: self._counter(1))
    num_prompt_tokens = property(lambda self: self._counter(2))
    num_decode_tokens = property(lambda self: self._counter(3))

    def _queue(self, which: int) -> List[int]:
        n = self._counter(4 + which)
        buf = np.zeros(max(n, 1), dtype=np.int32)
        got = self._lib.mgpt_sched_queue(self._h, which, _p(buf), buf.size)
        return buf[:got].tolist()

    @property
    def waiting(self) -> List[int]:
        return self._queue(0)

    @property
    def running(self) -> List[int]:
        return self._queue(1)

    def info(self, rid: int) -> RequestInfo:
        buf = np.zeros(6, dtype=np.int32)
        if self._lib.mgpt_sched_request_info(self._h, rid, _p(buf)) != 0:
            raise KeyError(f"no request {rid}")
        return RequestInfo(int(buf[0]), FINISH_REASONS[int(buf[1])], int(buf[2]), int(buf[3]), int(buf[4]), int(buf[5]))

    def output(self, rid: int) -> List[int]:
        n = self.info(rid).output_len
        buf = np.zeros(max(n, 1), dtype=np.int32)
        got = self._lib.mgpt_sched_copy_output(self._h, rid, _p(buf), buf.size)
        return buf[:got].tolist()

    def forget_finished(self) -> None:
        """Drops the records of finished requests (not while tokens of planned decode steps are still
        to be handed in); their ids go to later requests."""
        self._lib.mgpt_sched_forget_finished(self._h)

    @property
    def num_records(self) -> int:
        """Request records held now: waiting, running, and finished ones not yet forgotten."""
        return int(self._lib.mgpt_sched_num_records(self._h))
