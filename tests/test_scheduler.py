"""The scheduler's decisions (no GPU, no model): what the reference's tests pin
(tests/test_scheduler.py:121-243, tests/test_paged.py:107-143) and what is new here: prompt
portions under a token budget, mixed steps, and what happens when pages run out."""

import random

import numpy as np
import pytest

from mini_gpt_inference_amd.cache.manager import CacheManager, GroupGeometry
from mini_gpt_inference_amd.engine.scheduler import FINISHED, RUNNING, WAITING, Scheduler, SchedulerError


def make(num_pages, page_size, max_batch, budget=64, chunk=0, mixed=True, max_positions=1024, spare_asker=False):
    cm = CacheManager([GroupGeometry(page_size, num_pages, 0)], max_batch)
    return cm, Scheduler(cm, max_batch, budget, chunk, mixed, max_positions, spare_asker)


def step(sched, token=lambda rid, idx: 100 + idx):
    """Schedules one step and commits made-up tokens.  Returns (entries, outputs)."""
    sched.schedule()
    entries = sched.entries()
    toks = [token(e.request, sched.info(e.request).output_len) for e in entries if e.sample]
    outs = sched.commit(np.array(toks, dtype=np.int32))
    return entries, outs


def test_admits_up_to_max_batch_size():
    cm, s = make(100, 4, max_batch=2, mixed=False)
    for _ in range(3):
        s.add_request(list(range(4)), 10)
    n, r, m = s.schedule()
    assert (n, r, m) == (8, 2, 2) and len(s.waiting) == 1 and len(s.running) == 2


def test_decodes_when_nothing_is_admitted_and_prompts_go_first():
    cm, s = make(100, 4, max_batch=2, mixed=False)
    r0 = s.add_request(list(range(4)), 10)
    ents, _ = step(s)
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(r0, 0, 4, True)]
    ents, _ = step(s)
    assert [(e.request, e.ctx, e.q_len) for e in ents] == [(r0, 4, 1)]
    # a new arrival's prompt beats decoding of the running set (reference: prefill priority)
    r1 = s.add_request(list(range(4)), 10)
    ents, _ = step(s)
    assert [e.request for e in ents] == [r1]


def test_mixed_step_holds_decode_tokens_beside_a_prompt():
    cm, s = make(100, 4, max_batch=4, mixed=True)
    r0 = s.add_request(list(range(4)), 10)
    step(s)
    r1 = s.add_request(list(range(6)), 10)
    ents, _ = step(s)
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(r0, 4, 1, True), (r1, 0, 6, True)]
    assert s.num_decode_tokens == 1 and s.num_prompt_tokens == 10


def test_head_of_line_blocking():
    # reference tests/test_scheduler.py:159-168, with a head that fits the pool but not right now
    cm, s = make(3, 4, max_batch=10, mixed=False)
    first = s.add_request(list(range(8)), 2)   # 2 pages
    step(s)
    blocked = s.add_request(list(range(8)), 2)    # needs 2 pages, 1 free: waits
    behind = s.add_request([1, 2], 2)             # would fit, but is behind it
    ents, _ = step(s)
    assert [e.request for e in ents] == [first]   # nothing admitted: the running request decodes
    assert s.waiting == [blocked, behind]
    # nothing running and the head does not fit: an empty step, as the reference's ([], False)
    cm, s = make(3, 4, max_batch=10, mixed=False)
    a = s.add_request(list(range(8)), 2)
    slot = cm.acquire_slot()
    cm.reserve(slot, 8)                           # someone else holds 2 of the 3 pages
    assert s.schedule() == (0, 0, 0) and s.waiting == [a]


def test_nothing_to_do_returns_an_empty_step():
    cm, s = make(1, 4, max_batch=2, mixed=False, max_positions=16)
    a = s.add_request(list(range(4)), 1)
    step(s)
    assert not s.has_work()
    assert s.schedule() == (0, 0, 0)


def test_prompt_portions_under_a_budget_and_a_chunk():
    cm, s = make(100, 4, max_batch=4, budget=16, chunk=6, mixed=True)
    a = s.add_request(list(range(20)), 3)
    b = s.add_request(list(range(9)), 3)
    ents, outs = step(s)
    # a takes a chunk of 6, b a chunk of 6; neither is complete, nothing is sampled
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(a, 0, 6, False), (b, 0, 6, False)]
    assert outs == [] and s.info(a).num_computed == 6
    ents, outs = step(s)
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(a, 6, 6, False), (b, 6, 3, True)]
    assert [o[0] for o in outs] == [b]
    ents, _ = step(s)     # b decodes (1 token), a continues with a chunk
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(b, 9, 1, True), (a, 12, 6, False)]
    ents, _ = step(s)
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(b, 10, 1, True), (a, 18, 2, True)]
    # the budget cuts a portion short: 16 tokens a step
    cm, s = make(100, 4, max_batch=4, budget=16, chunk=0, mixed=True)
    a = s.add_request(list(range(20)), 2)
    ents, _ = step(s)
    assert [(e.ctx, e.q_len, e.sample) for e in ents] == [(0, 16, False)]
    ents, _ = step(s)
    assert [(e.ctx, e.q_len, e.sample) for e in ents] == [(16, 4, True)]


def test_finish_on_length_and_on_eot_frees_in_the_same_step():
    cm, s = make(10, 4, max_batch=4)
    a = s.add_request([1, 2, 3], 2)
    b = s.add_request([1, 2, 3], 30, eot=7)
    _, outs = step(s, token=lambda rid, idx: 7 if rid == b and idx == 1 else 5)
    assert outs == [(a, 5, False, None), (b, 5, False, None)]
    _, outs = step(s, token=lambda rid, idx: 7 if rid == b and idx == 1 else 5)
    # the eot token is appended and returned (reference engine.py:164,177-183)
    assert outs == [(a, 5, True, "length"), (b, 7, True, "eot")]
    assert s.output(b) == [5, 7] and s.info(a).status == FINISHED
    assert cm.num_free_pages() == 10 and cm.num_free_slots == 4 and not s.has_work()


def test_pages_run_out_newest_is_evicted_to_the_front_and_recomputed():
    # reference tests/test_paged.py:107-143: page size 2, 4 pages, prompts of 2, 4 new tokens each
    cm, s = make(4, 2, max_batch=2, mixed=True, max_positions=32)
    a = s.add_request([1, 2], 4)
    b = s.add_request([4, 5], 4)
    log = []
    seen = {}
    for _ in range(40):
        if not s.has_work():
            break
        ents, outs = step(s, token=lambda rid, idx: 10 * (rid + 1) + idx)
        log.append([(e.request, e.ctx, e.q_len) for e in ents])
        for rid, tok, fin, why in outs:
            seen.setdefault(rid, []).append(tok)
        assert cm.check() == 0
    assert not s.has_work()
    assert s.num_preemptions == 1
    # each output index was sampled exactly once, also for the evicted request
    assert seen[a] == [10, 11, 12, 13] and seen[b] == [20, 21, 22, 23]
    assert cm.num_free_pages() == 4
    # both prompts, then two decode steps for both (positions 2 and 3 share each one's second page)...
    assert log[0] == [(a, 0, 2), (b, 0, 2)]
    assert log[1] == [(a, 2, 1), (b, 2, 1)] and log[2] == [(a, 3, 1), (b, 3, 1)]
    # ...then both need a third page (position 4): a (older) keeps going, b (newest) is evicted
    evicted_at = next(i for i, ents in enumerate(log) if [e[0] for e in ents] == [a])
    assert log[evicted_at] == [(a, 4, 1)]
    # when a is done, b comes back as one portion of prompt + outputs, from position 0
    back = next(ents for ents in log[evicted_at:] if ents and ents[0][0] == b)
    assert back == [(b, 0, 2 + 3)]       # its prompt and the three tokens it had sampled


def test_evicted_request_goes_to_the_front_of_waiting():
    # after reference tests/test_scheduler.py:185-207 (there: 2 pages, which a single request of
    # this length could never finish in; such a request is refused here)
    cm, s = make(3, 4, max_batch=2, mixed=False, max_positions=64)
    old = s.add_request(list(range(4)), 5)
    new = s.add_request(list(range(4)), 5)
    later = s.add_request(list(range(4)), 5)     # not admitted: both places are taken
    step(s)                                       # both prompts (one page each)
    assert s.running == [old, new] and cm.num_free_pages() == 1
    ents, _ = step(s)                             # both at position 4: a second page each, one is free
    assert [e.request for e in ents] == [old]
    assert s.running == [old] and s.waiting == [new, later] and s.num_preemptions == 1
    assert len(cm.table(s.info(old).slot)) == 2   # the survivor got the freed page
    assert s.info(new).num_computed == 0 and s.info(new).output_len == 1 and s.info(new).status == WAITING


def test_the_references_victim_rule_can_be_switched_back_on():
    # The same three pages as above.  The older request takes the free page; then the newer one asks.
    # The reference (scheduler.py:66-82) never evicts the one that asks while another runs, so the
    # older request goes and the newer keeps decoding; both finish, and no page is lost.
    cm, s = make(3, 4, max_batch=2, mixed=False, max_positions=64, spare_asker=True)
    old = s.add_request(list(range(4)), 5)
    new = s.add_request(list(range(4)), 5)
    step(s)
    assert s.running == [old, new] and cm.num_free_pages() == 1
    ents, _ = step(s)
    assert [e.request for e in ents] == [new]
    assert s.running == [new] and s.waiting == [old] and s.num_preemptions == 1
    assert len(cm.table(s.info(new).slot)) == 2
    assert s.info(old).num_computed == 0 and s.info(old).status == WAITING
    # the last one running still gives way to nobody but itself: it is never asked to
    for _ in range(40):
        if not s.has_work():
            break
        step(s)
        assert cm.check() == 0
    assert not s.has_work() and cm.num_free_pages() == 3
    assert len(s.output(old)) == 5 and len(s.output(new)) == 5


def test_requests_that_can_never_run_are_refused():
    cm, s = make(4, 4, max_batch=2, max_positions=32)
    with pytest.raises(SchedulerError, match="empty"):
        s.add_request([], 4)
    with pytest.raises(SchedulerError, match="block_size"):       # reference engine.py:83-88
        s.add_request(list(range(30)), 3)
    with pytest.raises(SchedulerError, match="whole pool"):
        s.add_request(list(range(10)), 8)                          # 17 cached tokens > 4 pages of 4
    assert s.add_request(list(range(10)), 7) >= 0                  # 16 cached tokens: exactly the pool


def test_cancel():
    cm, s = make(10, 4, max_batch=1)
    r0 = s.add_request(list(range(4)), 5)
    r1 = s.add_request(list(range(4)), 5)
    step(s)
    assert s.running == [r0] and s.waiting == [r1] and cm.num_free_pages() == 9
    assert s.cancel(r1) and s.waiting == [] and cm.num_free_pages() == 9
    assert s.cancel(r0) and s.running == [] and cm.num_free_pages() == 10
    assert s.info(r0).finish_reason == "cancelled" and s.info(r0).status == FINISHED
    assert not s.cancel(r0) and not s.cancel(12345)


@pytest.mark.parametrize("mixed,chunk", [(True, 0), (True, 5), (False, 0), (False, 7)])
def test_random_load_keeps_every_invariant(mixed, chunk):
    rng = random.Random(1234 + chunk)
    cm, s = make(24, 4, max_batch=5, budget=32, chunk=chunk, mixed=mixed, max_positions=64)
    want, got, arrivals = {}, {}, 0
    for it in range(2000):
        if arrivals < 40 and rng.random() < 0.3:
            prompt = [rng.randrange(50) for _ in range(rng.randint(1, 30))]
            rid = s.add_request(prompt, rng.randint(1, 12))
            want[rid] = None
            got[rid] = []
            arrivals += 1
        if not s.has_work():
            if arrivals >= 40:
                break
            continue
        n, r, m = s.schedule()
        ents = s.entries()
        assert n <= 32 and r <= 5 and len({e.request for e in ents}) == len(ents)
        for e in ents:
            info = s.info(e.request)
            assert info.status == RUNNING
            assert e.ctx == info.num_computed                       # next position == tokens cached
            total = info.prompt_len + info.output_len
            assert 1 <= e.q_len <= total - e.ctx and e.sample == (e.ctx + e.q_len == total)
            assert len(cm.table(info.slot)) * 4 >= e.ctx + e.q_len   # pages are there before the step
        outs = s.commit(np.array([len(got[e.request]) for e in ents if e.sample], dtype=np.int32))
        for rid, tok, fin, why in outs:
            assert tok == len(got[rid])          # each output index exactly once, in order
            got[rid].append(tok)
        assert cm.check() == 0
    assert not s.has_work() and arrivals == 40
    assert all(s.info(rid).status == FINISHED and s.info(rid).finish_reason == "length" for rid in want)
    assert cm.num_free_pages() == 24 and cm.num_free_slots == 5


def test_burst_is_planned_only_when_nothing_else_is_pending_and_ends_on_the_end_token():
    cm, s = make(20, 4, max_batch=4, max_positions=64)
    a = s.add_request([1, 2, 3], 10, eot=7)
    b = s.add_request([1, 2, 3, 4, 5], 6)
    assert s.plan_burst(8) == 0                  # nobody is running yet
    step(s)                                      # both prompts, one token each
    c = s.add_request([9], 5)
    assert s.plan_burst(8) == 0                  # somebody waits
    step(s)                                      # c's prompt beside the decode tokens of a and b
    free_before = cm.num_free_pages()
    k = s.plan_burst(8)
    # a has 8 tokens left, b 4, c 4: the burst stops at the first length limit
    assert k == 4
    ents = s.entries()
    assert [(e.request, e.ctx, e.q_len, e.sample) for e in ents] == [(a, 4, 1, True), (b, 6, 1, True), (c, 1, 1, True)]
    for e in ents:       # pages for all four tokens are held before the burst starts
        assert len(cm.table(s.info(e.request).slot)) * 4 >= e.ctx + k
    assert cm.num_free_pages() <= free_before
    # a meets its end token in the burst's second step: what came after is dropped
    tokens = np.array([[5, 5, 5], [7, 5, 5], [6, 5, 5], [6, 5, 5]], dtype=np.int32)
    outs = s.commit_burst(tokens, k)
    assert [o for o in outs if o[0] == a] == [(a, 5, False, None), (a, 7, True, "eot")]
    assert [o[1:] for o in outs if o[0] == b] == [(5, False, None)] * 3 + [(5, True, "length")]
    assert s.output(a) == [100, 101, 5, 7] and s.info(b).status == FINISHED and s.info(c).status == FINISHED
    assert not s.has_work() and cm.num_free_pages() == 20 and cm.check() == 0


def test_a_burst_handed_in_in_stretches_ends_like_one_handed_in_whole():
    """The device is still at work on a burst's later steps when the first ones' tokens come back:
    the scheduler takes them stretch by stretch, a request that met its end token in an earlier
    stretch is passed over in the later ones, and entries last until the final stretch."""
    results = []
    for cuts in ([4], [1, 3], [2, 1, 1]):
        cm, s = make(20, 4, max_batch=4, max_positions=64)
        a = s.add_request([1, 2, 3], 10, eot=7)
        b = s.add_request([1, 2, 3, 4, 5], 5)
        step(s)
        assert s.plan_burst(8) == 4
        tokens = np.array([[5, 5], [7, 5], [6, 5], [6, 5]], dtype=np.int32)
        outs, first = [], 0
        for n in cuts:
            assert len(s.entries()) == 2
            outs += s.commit_burst(tokens[first:first + n], n, last=first + n == 4)
            first += n
        assert len(s.entries()) == 0
        results.append((outs, s.output(a), s.output(b), cm.num_free_pages(), cm.check()))
        assert s.info(a).status == FINISHED and s.info(b).status == FINISHED and not s.has_work()
    assert results[0] == results[1] == results[2]
    assert results[0][1] == [100, 5, 7] and results[0][3] == 20 and results[0][4] == 0


def test_a_burst_can_be_planned_ahead_of_one_whose_tokens_are_not_all_in():
    """The device runs the next burst right behind the last one: the scheduler plans it from where
    that one will end, reserves its pages, and refuses once a request of the last one has ended."""
    cm, s = make(40, 4, max_batch=4, max_positions=64)
    a = s.add_request([1, 2, 3], 20, eot=7)
    b = s.add_request([1, 2, 3, 4, 5], 14)
    step(s)
    assert s.plan_burst(4) == 4                       # steps 0..3: a at 3.., b at 5..
    toks = np.full((4, 2), 5, dtype=np.int32)
    s.commit_burst(toks[:2], 2, last=False)           # two steps are in, two are not
    assert s.plan_burst(4) == 4                       # ahead: starts where the first burst ends
    ents = s.entries()
    assert [(e.request, e.ctx) for e in ents] == [(a, 3 + 4), (b, 5 + 4)]
    for e in ents:                                    # pages up to the end of the second burst
        assert len(cm.table(s.info(e.request).slot)) * 4 >= e.ctx + 4
    with pytest.raises(Exception):                    # no other scheduling while steps are out
        s.schedule()
    s.commit_burst(toks[2:], 2, last=True)            # the first burst's last stretch: entries stay
    assert len(s.entries()) == 2
    assert s.plan_burst(8) == 5                       # b has 14 - 5 - 4 = 5 left once the second burst is in
    outs = s.commit_burst(toks, 4, last=True)
    assert len(outs) == 8 and len(s.entries()) == 2   # the third burst is still out
    # a meets its end token in the third burst's first step: no burst goes on behind that
    toks5 = np.full((5, 2), 5, dtype=np.int32)
    toks5[0, 0] = 7
    s.commit_burst(toks5[:1], 1, last=False)
    assert s.info(a).status == FINISHED
    assert s.plan_burst(8) == 0
    outs = s.commit_burst(toks5[1:], 4, last=True)
    assert [o[0] for o in outs] == [b] * 4 and outs[-1][2:] == (True, "length") and len(s.entries()) == 0
    assert s.output(a) == [100] + [5] * 8 + [7]
    assert s.output(b) == [100] + [5] * 13
    assert not s.has_work() and cm.num_free_pages() == 40 and cm.check() == 0


def test_filling_a_burst_planned_ahead_reads_no_token_the_host_does_not_have():
    """The first token of a burst planned ahead exists on the device only: the filled step names
    position, cache slot and block table for it and leaves its token id at zero."""
    import torch
    from mini_gpt_inference_amd.engine.step import StepArena
    cm, s = make(40, 4, max_batch=4, max_positions=64)
    a = s.add_request([1, 2, 3], 20)
    step(s)
    assert s.plan_burst(4) == 4
    arena = StepArena(4, 4, 4, 1, 16, torch.device("cpu"))
    s.fill(arena)
    assert arena.h["token_ids"][0] == 100 and arena.h["positions"][0] == 3
    assert s.plan_burst(4) == 4                     # ahead of the four steps that are still out
    arena.h["token_ids"][:] = -7
    s.fill(arena)
    slot = s.info(a).slot
    assert arena.h["token_ids"][0] == 0 and arena.h["positions"][0] == 7 and arena.h["seq_lens"][0] == 8
    assert arena.h["slot_mapping"][0] == cm.table(slot)[7 // 4] * 4 + 7 % 4
    assert list(arena.h["block_tables"][:3]) == cm.table(slot)[:3]
    s.commit_burst(np.full((8, 1), 5, dtype=np.int32), 8)
    assert s.output(a) == [100] + [5] * 8


def test_burst_needs_pages_for_every_step_or_does_not_start():
    cm, s = make(4, 4, max_batch=2, max_positions=64)
    a = s.add_request([1, 2, 3], 12)
    b = s.add_request([1, 2, 3], 12)
    step(s)
    free = cm.num_free_pages()
    assert s.plan_burst(8) == 0 and cm.num_free_pages() == free     # 2 free pages, 4 would be needed
    assert s.plan_burst(2) == 2                                      # two more tokens each fit


def test_a_scheduler_that_serves_for_long_holds_only_its_live_requests():
    """Finished requests are forgotten for good: their records go and their ids are given to later
    requests, so the number of records follows the live requests, not the requests ever served.  A
    request's default sampling stream is its place in the order of arrival, not its id."""
    cm, s = make(32, 4, max_batch=4)
    seen_ids = set()
    for wave in range(50):
        ids = [s.add_request([1, 2, 3], 2) for _ in range(3)]
        seen_ids.update(ids)
        assert s.num_records <= 3 + 3                       # this wave's and, before forgetting, the last one's
        while s.has_work():
            step(s)
        assert all(s.info(i).status == FINISHED and s.output(i) == [100, 101] for i in ids)
        s.forget_finished()
        assert s.num_records == 0
        for i in ids:
            with pytest.raises(KeyError):
                s.info(i)
    assert len(seen_ids) <= 6, "ids of forgotten requests were not used again"
    assert cm.num_free_pages() == 32 and cm.check() == 0
    # a forgotten id among live ones: the others stay what they were
    a, b = s.add_request([5] * 5, 3), s.add_request([6] * 2, 1)
    while s.info(b).status != FINISHED:
        step(s)
    s.forget_finished()
    c = s.add_request([7] * 3, 2)
    assert c == b and s.info(a).status == RUNNING and s.info(c).status == WAITING and s.info(c).prompt_len == 3
    while s.has_work():
        step(s)
    assert s.output(a) == [100, 101, 102] and s.output(c) == [100, 101]


def test_records_are_kept_while_a_planned_burst_is_not_all_handed_in():
    cm, s = make(32, 4, max_batch=2)
    ids = [s.add_request([1, 2, 3], 9, eot=7) for _ in range(2)]
    step(s)
    step(s)
    k = s.plan_burst(4)
    assert k == 4
    tokens = np.full((4, 2), 50, dtype=np.int32)
    tokens[1, 0] = 7                                   # request 0 meets its end token in the burst's second step
    s.commit_burst(tokens[:2], 2, last=False)
    assert s.info(ids[0]).status == FINISHED
    s.forget_finished()                                # refused: two steps of the burst are still to come
    assert s.num_records == 2 and s.info(ids[0]).status == FINISHED
    s.commit_burst(tokens[2:], 2, last=True)
    s.forget_finished()
    assert s.num_records == 1 and s.info(ids[1]).status == RUNNING


@pytest.mark.parametrize("seed", range(4))
def test_random_load_with_forgetting_at_random_times(seed):
    """Arrivals, steps, bursts, cancels and forget_finished in random order: ids are given out again,
    and still every request gets its own outputs, each output index once and in order, nothing of a
    forgotten request comes back, and the records follow the live requests."""
    rng = random.Random(99 + seed)
    cm, s = make(28, 4, max_batch=4, budget=24, chunk=6, mixed=True, max_positions=64)
    live = {}            # id -> (serial number of the request, its output length so far, max_tokens)
    serial = done = 0
    for it in range(3000):
        roll = rng.random()
        if roll < 0.25 and serial < 120:
            rid = s.add_request([rng.randrange(50) for _ in range(rng.randint(1, 20))], rng.randint(1, 10))
            assert rid not in live, "an id in use was given out again"
            live[rid] = [serial, 0, None]
            serial += 1
        elif roll < 0.30 and live:
            rid = rng.choice(list(live))
            if s.info(rid).status != FINISHED:
                assert s.cancel(rid)
        elif roll < 0.40:
            before = s.num_records
            s.forget_finished()
            for rid in list(live):
                try:
                    s.info(rid)
                except KeyError:
                    del live[rid]
                    done += 1
            assert s.num_records == len(live) <= before
        if not s.has_work():
            continue
        k = s.plan_burst(4) if rng.random() < 0.3 else 0
        if k >= 2:
            ents = s.entries()
            toks = np.array([[live[e.request][0] * 100 + live[e.request][1] + j for e in ents] for j in range(k)],
                            dtype=np.int32)
            outs = s.commit_burst(toks, k)
        else:
            s.schedule()
            ents = s.entries()
            outs = s.commit(np.array([live[e.request][0] * 100 + live[e.request][1] for e in ents if e.sample],
                                     dtype=np.int32))
        for rid, tok, fin, why in outs:
            rec = live[rid]
            assert tok == rec[0] * 100 + rec[1], "a token of another request, or out of order"
            rec[1] += 1
        assert cm.check() == 0
    while s.has_work():
        s.schedule()
        ents = s.entries()
        for rid, tok, fin, why in s.commit(np.array([live[e.request][0] * 100 + live[e.request][1]
                                                     for e in ents if e.sample], dtype=np.int32)):
            live[rid][1] += 1
    s.forget_finished()
    assert s.num_records == 0 and serial > 50 and cm.num_free_pages() == 28 and cm.num_free_slots == 4
