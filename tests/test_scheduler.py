"""The scheduler's decisions, driven with made-up sampled tokens (no model, no GPU)."""
import random

import pytest
import torch

from spite_amd.cache.paged import PagedCache
from spite_amd.engine.scheduler import Scheduler, SchedulerError
from spite_amd.parts.base import CacheNeed, KVNeed

FULL = CacheNeed(kv=KVNeed(2, 16, "full"))
CHUNK32 = CacheNeed(kv=KVNeed(2, 16, "chunk", 32))


def make(pages=16, page_size=16, max_requests=4, budget=32, ctx=1 << 20, eos=(), needs=(CHUNK32, FULL)):
    c = PagedCache(list(needs), page_size, pages, max_requests, torch.float32, torch.device("cpu"), allocate=False)
    return c, Scheduler(c, budget, ctx, eos)


def shape(batch):
    return [(b.request_id, b.start, len(b.tokens), b.wants_logits) for b in batch]


def run(s, next_token=lambda rid, k: 100 + k, max_steps=10_000):
    """Drives to the end; returns {request: emitted tokens}, {request: reason}."""
    toks, why, k = {}, {}, 0
    for _ in range(max_steps):
        if s.active_count() == 0:
            return toks, why
        batch = s.schedule()
        outs = s.update([next_token(b.request_id, k) for b in batch if b.wants_logits])
        k += 1
        for o in outs:
            if o.token >= 0:
                toks.setdefault(o.request_id, []).append(o.token)
            if o.done:
                why[o.request_id] = o.finish_reason
    raise AssertionError("scheduler did not finish")


def test_prompt_is_cut_into_portions_under_the_budget():
    c, s = make(budget=32)
    a = s.submit(list(range(70)), 2)
    assert shape(s.schedule()) == [(a, 0, 32, False)]
    s.update([])
    assert shape(s.schedule()) == [(a, 32, 32, False)]
    s.update([])
    assert shape(s.schedule()) == [(a, 64, 6, True)]
    outs = s.update([7])
    assert [(o.token, o.done) for o in outs] == [(7, False)]
    b = s.schedule()
    assert shape(b) == [(a, 70, 1, True)] and b[0].tokens == [7]         # the sampled token is fed next
    outs = s.update([8])
    assert [(o.token, o.done, o.finish_reason) for o in outs] == [(8, True, "MaxTokens")]
    assert s.active_count() == 0 and c.free_slots() == 4 and c.free_pages(0) == 16 and c.free_pages(1) == 16
    c.check()


def test_decodes_come_first_then_prompts_under_way_then_new_requests():
    c, s = make(budget=16)
    a = s.submit([1] * 4, 8)
    s.schedule(); s.update([50])                                        # a decodes from now on
    b = s.submit([2] * 40, 8)
    assert shape(s.schedule()) == [(a, 4, 1, True), (b, 0, 15, False)]  # the budget's rest goes to b
    s.update([51])
    d = s.submit([3] * 3, 8)
    # a: 1 token, b: continues with 15 - nothing is left for d, which waits its turn
    assert shape(s.schedule()) == [(a, 5, 1, True), (b, 15, 15, False)]
    s.update([52])
    assert shape(s.schedule()) == [(a, 6, 1, True), (b, 30, 10, True), (d, 0, 3, True)]
    assert s.n_running == 3 and s.n_waiting == 0


def test_portions_shrink_to_one_token():
    c, s = make(budget=4)
    a = s.submit([1] * 2, 5)
    b = s.submit([2] * 2, 5)
    e = s.submit([3] * 9, 5)
    assert shape(s.schedule()) == [(a, 0, 2, True), (b, 0, 2, True)]
    s.update([9, 9])
    assert shape(s.schedule()) == [(a, 2, 1, True), (b, 2, 1, True), (e, 0, 2, False)]
    s.update([9, 9])
    assert shape(s.schedule())[2] == (e, 2, 2, False)


def test_finishing_reasons_and_tokens_that_are_not_emitted():
    c, s = make(eos=(0,))
    a = s.submit([5, 6], 10)
    b = s.submit([5, 6], 10, stop_tokens=[77])
    d = s.submit([5, 6], 3)
    feed = {a: [11, 12, 0, 99], b: [11, 77, 99], d: [11, 12, 13, 99]}
    counters = {a: 0, b: 0, d: 0}
    def nxt(rid, k):
        counters[rid] += 1
        return feed[rid][counters[rid] - 1]
    toks, why = run(s, nxt)
    assert toks == {a: [11, 12], b: [11], d: [11, 12, 13]}              # eos and stop tokens are not emitted
    assert why == {a: "EosToken", b: "StopToken", d: "MaxTokens"}
    assert c.free_slots() == 4
    c.check()


def test_context_limit():
    c, s = make(ctx=6)
    with pytest.raises(SchedulerError, match="longer than the context limit"):
        s.submit([1] * 7, 4)
    a = s.submit([1] * 4, 10)
    toks, why = run(s)
    assert len(toks[a]) == 2 and why[a] == "ContextLimit"               # 4 + 2 = 6 positions


def test_rejections():
    c, s = make(pages=2, page_size=16)
    with pytest.raises(SchedulerError, match="empty prompt"):
        s.submit([], 4)
    with pytest.raises(SchedulerError, match="pages"):
        s.submit([1] * 40, 4)                                           # 3 pages of the full group, the pool has 2
    assert s.active_count() == 0


def test_no_admission_while_pages_are_short():
    c, s = make(pages=4, page_size=16, budget=64, needs=(FULL,))
    a = s.submit([1] * 40, 50)                                          # 3 pages
    b = s.submit([2] * 30, 50)                                          # 2 pages: does not fit beside a
    assert shape(s.schedule()) == [(a, 0, 40, True)]
    assert s.n_waiting == 1
    s.update([9])
    assert shape(s.schedule()) == [(a, 40, 1, True)]                    # b still waits: 1 page free, needs 2
    s.update([9])


def test_preemption_of_the_request_admitted_last():
    c, s = make(pages=4, page_size=16, budget=64, needs=(FULL,))
    a = s.submit([1] * 30, 100)                                         # 2 pages, grows
    b = s.submit([2] * 20, 100)                                         # 2 pages
    assert shape(s.schedule()) == [(a, 0, 30, True), (b, 0, 20, True)]
    s.update([9, 9])
    assert c.free_pages(0) == 0
    steps = 0
    while s.n_preemptions == 0:
        batch = s.schedule()
        s.update([9] * sum(x.wants_logits for x in batch))
        steps += 1
        assert steps < 40
    # a reached position 32 and needed a third page: b, admitted last, gave way
    info_b, info_a = s.request_info(b), s.request_info(a)
    assert info_b["n_preempted"] == 1 and info_b["slot"] == -1 and info_b["n_computed"] == 0
    assert info_a["n_preempted"] == 0 and s.n_waiting == 1
    n_gen_b = info_b["n_generated"]
    assert n_gen_b >= 1
    c.check()
    # b comes back when pages are free and is computed again from its start, all its tokens
    while s.n_waiting:
        batch = s.schedule()
        s.update([9] * sum(x.wants_logits for x in batch))
        if s.request_info(a) is None:
            break
    toks, why = run(s)
    c.check()
    assert c.free_slots() == 4 and c.free_pages(0) == 4


def test_a_lone_request_that_cannot_grow_fails_with_out_of_pages():
    c, s = make(pages=2, page_size=16, budget=64, needs=(FULL,))
    a = s.submit([1] * 30, 100)
    toks, why = run(s)
    assert why[a] == "OutOfPages" and len(toks[a]) == 3                 # positions 30, 31 fit; 32 needs a third page
    assert c.free_pages(0) == 2 and c.free_slots() == 4


def test_chunked_group_rolls_on_with_a_small_pool():
    # the chunked group needs a chunk and a portion, not the whole prompt
    c = PagedCache([CHUNK32], 16, 4, 2, torch.float32, torch.device("cpu"), allocate=False)
    s = Scheduler(c, 16, 1 << 20, ())
    a = s.submit([1] * 200, 4)
    toks, why = run(s)
    assert why[a] == "MaxTokens" and len(toks[a]) == 4
    c.check()


def test_cancel():
    c, s = make()
    a, b = s.submit([1] * 5, 5), s.submit([2] * 5, 5)
    s.schedule(); s.update([9, 9])
    assert s.cancel(a) and not s.cancel(a)
    toks, why = run(s)
    assert list(why) == [b] and c.free_slots() == 4
    c.check()


@pytest.mark.parametrize("seed", range(5))
def test_random_arrivals_with_tiny_pools_finish_every_request(seed):
    rnd = random.Random(seed)
    c, s = make(pages=rnd.choice([5, 8, 12]), page_size=rnd.choice([4, 16]), max_requests=3, budget=rnd.choice([6, 24]),
                eos=(0,))
    expect, done, emitted = {}, {}, {}
    pending = 12
    for step in range(5000):
        if pending and rnd.random() < 0.3:
            n = rnd.choice([1, 3, 9, 20, 33])
            try:
                rid = s.submit([rnd.randrange(1, 50) for _ in range(n)], rnd.choice([1, 4, 12]))
                expect[rid] = True
            except SchedulerError:
                pass
            pending -= 1
        if s.active_count() == 0:
            if not pending:
                break
            continue
        batch = s.schedule()
        ids = [b.request_id for b in batch]
        assert len(ids) == len(set(ids)) and sum(len(b.tokens) for b in batch) <= s.max_batch_tokens
        for b in batch:
            assert b.start == c.cached(b.slot)
        outs = s.update([rnd.choice([0, 5, 6, 7, 8, 9, 10, 11]) for b in batch if b.wants_logits])
        for o in outs:
            if o.done:
                done[o.request_id] = o.finish_reason
        c.check()
    assert set(done) == set(expect)
    assert set(done.values()) <= {"EosToken", "MaxTokens", "OutOfPages"}
    assert c.free_slots() == 3 and all(c.free_pages(g) == c.total_pages(g) for g in range(2))
