"""The cache manager (no GPU): vectors of the reference's allocator tests, windows, request slots,
and random orders of requests under which no page may be lost, held twice or freed twice."""

import random

import numpy as np
import pytest

from mini_gpt_inference_amd.cache.manager import CacheError, CacheManager, GroupGeometry


def _one(num_pages, page_size, max_requests=8, window=0):
    return CacheManager([GroupGeometry(page_size, num_pages, window)], max_requests)


def test_allocate_tracks_free_count_and_is_idempotent():
    cm = _one(10, 4)                      # reference tests/test_scheduler.py:25-39
    s = cm.acquire_slot()
    assert cm.reserve(s, 9)
    assert len(cm.table(s)) == 3 and cm.num_free_pages() == 7
    assert cm.reserve(s, 9)
    assert len(cm.table(s)) == 3 and cm.num_free_pages() == 7


def test_growth_only_at_a_page_boundary():
    cm = _one(10, 4)                      # tests/test_scheduler.py:42-54
    s = cm.acquire_slot()
    assert cm.reserve(s, 3) and len(cm.table(s)) == 1
    assert cm.reserve(s, 3 + 1) and len(cm.table(s)) == 1      # position 3 still fits
    assert cm.reserve(s, 4 + 1) and len(cm.table(s)) == 2      # position 4 needs a second page


def test_exhausted_pool_returns_false_without_change():
    cm = _one(1, 4)                       # tests/test_scheduler.py:57-65
    s = cm.acquire_slot()
    assert cm.reserve(s, 4) and cm.num_free_pages() == 0
    assert not cm.reserve(s, 5)
    assert len(cm.table(s)) == 1 and cm.check() == 0


def test_can_allocate_and_free():
    cm = _one(2, 4)                       # tests/test_scheduler.py:68-80
    assert cm.can_allocate(8) and not cm.can_allocate(9)
    s = cm.acquire_slot()
    cm.reserve(s, 8)
    assert cm.free_slot(s) and cm.num_free_pages() == 2
    assert not cm.free_slot(s)            # freed twice: refused, nothing changes
    assert cm.check() == 0


def test_lifo_order_of_pages_and_slots():
    cm = _one(6, 2)
    a, b = cm.acquire_slot(), cm.acquire_slot()
    assert (a, b) == (0, 1)
    cm.reserve(a, 4)
    assert cm.table(a) == [5, 4]          # taken from the end of the list (reference paged.py:63)
    cm.reserve(b, 2)
    cm.free_slot(a)
    c = cm.acquire_slot()
    assert c == a
    cm.reserve(c, 2)
    assert cm.table(c) == [4]             # the page freed last is used again first
    assert cm.check() == 0


def test_slots_run_out():
    cm = _one(4, 4, max_requests=2)
    a, b = cm.acquire_slot(), cm.acquire_slot()
    assert cm.acquire_slot() == -1 and cm.num_free_slots == 0
    cm.free_slot(a)
    assert cm.acquire_slot() == a


def test_window_group_gives_pages_back_as_the_window_passes():
    cm = CacheManager([GroupGeometry(4, 16, 0), GroupGeometry(4, 16, 6)], 4)
    s = cm.acquire_slot()
    assert cm.reserve(s, 20)
    assert cm.held_pages(s, 0) == 5 and cm.held_pages(s, 1) == 5
    # 13 tokens computed: the next query (position 13) sees keys 8..13 -> pages 0 and 1 are passed
    assert cm.release_passed(s, 13) == 2
    assert cm.table(s, 1)[:3] == [-1, -1, cm.table(s, 1)[2]] and cm.held_pages(s, 1) == 3
    assert cm.held_pages(s, 0) == 5       # the group that keeps all keys keeps them
    assert cm.release_passed(s, 13) == 0
    assert cm.num_free_pages(1) == 13 and cm.check() == 0
    cm.free_slot(s)
    assert cm.num_free_pages(0) == 16 and cm.num_free_pages(1) == 16 and cm.check() == 0


def test_reserve_is_all_or_nothing_across_groups():
    cm = CacheManager([GroupGeometry(4, 8, 0), GroupGeometry(4, 2, 0)], 4)
    s = cm.acquire_slot()
    assert not cm.reserve(s, 12)          # the second group has 2 pages, 3 are needed
    assert cm.num_free_pages(0) == 8 and cm.num_free_pages(1) == 2 and cm.table(s, 0) == []
    assert not cm.can_allocate(12) and cm.can_allocate(8)


def test_build_step_arrays():
    cm = _one(8, 4)
    a, b = cm.acquire_slot(), cm.acquire_slot()
    cm.reserve(a, 6)
    cm.reserve(b, 3)
    ta, tb = cm.table(a), cm.table(b)
    n_stride, r_stride, mb = 8, 4, 3
    pos, qr = np.zeros(n_stride, np.int32), np.zeros(n_stride, np.int32)
    cu, sl = np.zeros(r_stride + 1, np.int32), np.zeros(r_stride, np.int32)
    sm, bt = np.zeros(n_stride, np.int32), np.zeros(r_stride * mb, np.int32)
    n = cm.build_step([a, b], [4, 0], [2, 3], n_stride, r_stride, mb, pos, qr, cu, sl, sm, bt)
    assert n == 5
    assert pos.tolist() == [4, 5, 0, 1, 2, 0, 0, 0] and qr.tolist() == [0, 0, 1, 1, 1, -1, -1, -1]
    assert cu.tolist() == [0, 2, 5, 5, 5] and sl.tolist() == [6, 3, 0, 0]
    # slot = page * page_size + position % page_size (reference engine.py:123-125)
    assert sm.tolist() == [ta[1] * 4 + 0, ta[1] * 4 + 1, tb[0] * 4, tb[0] * 4 + 1, tb[0] * 4 + 2, -1, -1, -1]
    assert bt.reshape(r_stride, mb).tolist() == [ta + [-1], tb + [-1, -1], [-1] * 3, [-1] * 3]
    with pytest.raises(CacheError, match="no page"):
        cm.build_step([b], [3], [2], n_stride, r_stride, mb, pos, qr, cu, sl, sm, bt)


def test_random_orders_of_requests_lose_no_page():
    rng = random.Random(0)                # after tests/test_scheduler.py:83-104, with growth and windows
    cm = CacheManager([GroupGeometry(4, 64, 0), GroupGeometry(4, 64, 10)], 6)
    live = {}
    for i in range(3000):
        action = rng.choice(["new", "grow", "grow", "free"])
        if action == "new":
            s = cm.acquire_slot()
            if s >= 0:
                n = rng.randint(1, 40)
                if cm.reserve(s, n):
                    live[s] = n
                else:
                    cm.free_slot(s)
        elif action == "grow" and live:
            s = rng.choice(list(live))
            n = live[s] + rng.randint(1, 9)
            if cm.reserve(s, n):
                live[s] = n
                cm.release_passed(s, n)
        elif action == "free" and live:
            s = rng.choice(list(live))
            del live[s]
            assert cm.free_slot(s)
        assert cm.check() == 0, f"inconsistent after action {i} ({action})"
        for s, n in live.items():
            assert cm.held_pages(s, 0) == -(-n // 4)
            assert cm.held_pages(s, 1) <= -(-n // 4)
    for s in list(live):
        cm.free_slot(s)
    assert cm.num_free_pages(0) == 64 and cm.num_free_pages(1) == 64 and cm.num_free_slots == 6
    assert cm.check() == 0


def test_cache_groups_are_sized_by_bytes_so_that_each_holds_the_same_requests():
    """kv_cache_bytes is split over the groups by what a full-length request costs in each: a group
    with a window needs few pages per request, one with more heads costs more per page."""
    from types import SimpleNamespace as G
    from mini_gpt_inference_amd.cache.manager import CacheError, plan_group_pages
    full = G(n_kv_head=8, head_dim=64, window=0, n_pools=6)
    windowed = G(n_kv_head=2, head_dim=64, window=128, n_pools=2)
    assert plan_group_pages([full, windowed], 16, 777, None, 2, 1024) == [777, 777]       # the shorthand
    page_full, page_win = 6 * 2 * 8 * 16 * 64 * 2, 2 * 2 * 2 * 16 * 64 * 2
    per_request = 64 * page_full + 9 * page_win         # 1024 / 16 pages, and (128 + 16) / 16
    pages = plan_group_pages([full, windowed], 16, 777, 10 * per_request + 5, 2, 1024)
    assert pages == [640, 90]
    assert pages[0] * page_full + pages[1] * page_win <= 10 * per_request + 5
    one = plan_group_pages([full], 16, 1, 3 * 64 * page_full, 2, 1024)
    assert one == [192]
    assert plan_group_pages([full], 16, 1, 2 * 256 * (page_full * 2), 4, None) == [512]    # no bound on positions: 4096 tokens
    import pytest
    with pytest.raises(CacheError, match="does not hold one request"):
        plan_group_pages([full, windowed], 16, 1, per_request - 1, 2, 1024)
