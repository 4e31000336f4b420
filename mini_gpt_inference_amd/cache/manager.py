"""Python face of the C++ cache manager (csrc/host/cache_manager.h): pages per cache group,
a block table per request and group, and the request slots that index per-request state."""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np

from ..ops import library


@dataclass(frozen=True)
class GroupGeometry:
    page_size: int
    num_pages: int
    window: int = 0


class CacheError(RuntimeError):
    pass


NOMINAL_SPAN = 4096   # tokens a request is taken to hold where the model puts no bound on positions


def plan_group_pages(groups, page_size: int, num_blocks: int, kv_cache_bytes, itemsize: int,
                     max_positions=None) -> List[int]:
    """Pages of every cache group.  groups: the layout's CacheGroupSpec list (n_kv_head, head_dim,
    window, n_pools).  Without kv_cache_bytes every group gets num_blocks pages (the one-group
    shorthand, the reference's num_blocks).  With it the bytes are split so that every group holds
    the same number of full-length requests: a group's page costs n_pools * 2 * n_kv_head * page_size
    * head_dim * itemsize bytes, and a full-length request holds its whole span in a group that
    keeps all keys but only a window (and the page being written) in one that keeps a window."""
    if kv_cache_bytes is None:
        return [int(num_blocks)] * len(groups)
    span_all = int(max_positions) if max_positions else NOMINAL_SPAN
    page_bytes, pages_per_request = [], []
    for g in groups:
        page_bytes.append(g.n_pools * 2 * g.n_kv_head * page_size * g.head_dim * itemsize)
        span = min(g.window + page_size, span_all) if g.window else span_all
        pages_per_request.append(-(-span // page_size))
    per_request = sum(b * n for b, n in zip(page_bytes, pages_per_request))
    if per_request <= 0:
        return [1] * len(groups)
    requests = kv_cache_bytes / per_request
    if requests < 1.0:
        raise CacheError(f"kv_cache_bytes = {kv_cache_bytes} does not hold one request of full length "
                         f"({per_request} bytes over {len(groups)} cache groups)")
    return [max(n, int(requests * n)) for n in pages_per_request]


def _ip(a):
    """The address of an int32 array for the library; an address (int) passes through, which lets a
    caller that fills the same arrays at every step look them up once."""
    if isinstance(a, int):
        return a
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


class CacheManager:
    def __init__(self, groups: Sequence[GroupGeometry], max_requests: int) -> None:
        self._lib = library.host()
        self.groups = list(groups)
        self.max_requests = int(max_requests)
        n = len(self.groups)
        arr = lambda vals: (ctypes.c_int * n)(*vals)
        self._h = self._lib.mgpt_cache_create(n, arr([g.page_size for g in self.groups]),
                                              arr([g.num_pages for g in self.groups]),
                                              arr([g.window for g in self.groups]), self.max_requests)
        if not self._h:
            raise CacheError(library.host_error())

    def __del__(self) -> None:
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.mgpt_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    # request slots
    def acquire_slot(self) -> int:
        return self._lib.mgpt_cache_acquire_slot(self._h)

    def slot_live(self, slot: int) -> bool:
        return bool(self._lib.mgpt_cache_slot_live(self._h, slot))

    @property
    def num_free_slots(self) -> int:
        return self._lib.mgpt_cache_num_free_slots(self._h)

    # pages
    def pages_needed(self, n_tokens: int, group: int = 0) -> int:
        return self._lib.mgpt_cache_pages_needed(self._h, group, n_tokens)

    def can_allocate(self, n_tokens: int) -> bool:
        return bool(self._lib.mgpt_cache_can_allocate(self._h, n_tokens))

    def reserve(self, slot: int, n_tokens: int) -> bool:
        """Pages for positions [0, n_tokens) in every group; False (nothing changed) if they run out."""
        return bool(self._lib.mgpt_cache_reserve(self._h, slot, n_tokens))

    def release_passed(self, slot: int, n_computed: int) -> int:
        return self._lib.mgpt_cache_release_passed(self._h, slot, n_computed)

    def free_slot(self, slot: int) -> bool:
        return bool(self._lib.mgpt_cache_free_slot(self._h, slot))

    def num_free_pages(self, group: int = 0) -> int:
        return self._lib.mgpt_cache_num_free_pages(self._h, group)

    def held_pages(self, slot: int, group: int = 0) -> int:
        return self._lib.mgpt_cache_held_pages(self._h, slot, group)

    def table(self, slot: int, group: int = 0) -> List[int]:
        n = self._lib.mgpt_cache_table_len(self._h, slot, group)
        if n < 0:
            raise CacheError(f"slot {slot} is not live")
        buf = np.empty(max(n, 1), dtype=np.int32)
        got = self._lib.mgpt_cache_copy_table(self._h, slot, group, _ip(buf), buf.size)
        return buf[:got].tolist()

    def check(self) -> int:
        """0 when no page is lost, held twice or both held and free."""
        return self._lib.mgpt_cache_check(self._h)

    def build_step(self, slots: Sequence[int], ctx_lens: Sequence[int], q_lens: Sequence[int], n_stride: int,
                   r_stride: int, max_blocks: int, positions: np.ndarray, q_req: np.ndarray, cu_q: np.ndarray,
                   seq_lens: np.ndarray, slot_mapping: np.ndarray, block_tables: np.ndarray) -> int:
        """Fills the step's per-token and per-request arrays (int32 arrays of the strides' sizes, or
        their addresses, all six alike) and returns the number of tokens."""
        r = len(slots)
        mk = lambda v: np.ascontiguousarray(np.asarray(v, dtype=np.int32).reshape(-1))
        s, c, q = mk(slots), mk(ctx_lens), mk(q_lens)
        if r == 0:
            s = c = q = np.zeros(1, dtype=np.int32)
        g = len(self.groups)
        if not isinstance(positions, int):
            assert positions.size >= n_stride and q_req.size >= n_stride and cu_q.size >= r_stride + 1
            assert seq_lens.size >= r_stride and slot_mapping.size >= g * n_stride
            assert block_tables.size >= g * r_stride * max_blocks
        n = self._lib.mgpt_cache_build_step(self._h, r, _ip(s), _ip(c), _ip(q), n_stride, r_stride, max_blocks,
                                            _ip(positions), _ip(q_req), _ip(cu_q), _ip(seq_lens),
                                            _ip(slot_mapping), _ip(block_tables))
        if n == -1:
            raise CacheError("a token of the step has no page: reserve before stepping")
        if n == -2:
            raise CacheError("a block table is longer than max_blocks")
        if n < 0:
            raise CacheError(f"build_step refused its arguments ({n}) {library.host_error()}")
        return n
