"""The cache manager's books: pages per group, block tables, giving back and reuse, request
slots.  No GPU: the pools are not allocated, only accounted for."""
import random

import numpy as np
import pytest
import torch

from spite_amd.cache.paged import PagedCache, OutOfPages, CacheError
from spite_amd.parts.base import CacheNeed, KVNeed, StateNeed


def make(needs, page_size=16, pages=8, max_requests=4):
    return PagedCache(needs, page_size, pages, max_requests, torch.float32, torch.device("cpu"), allocate=False)


FULL = CacheNeed(kv=KVNeed(2, 16, "full"))
CHUNK32 = CacheNeed(kv=KVNeed(2, 16, "chunk", 32))
WIN20 = CacheNeed(kv=KVNeed(2, 16, "window", 20))


def test_reference_pool_vector():
    # crates/spite-kvcache/src/paged.rs:177-194: 8 blocks of 16; 16 commits -> 1 block used, 7 free; free_all -> 8
    c = make([FULL], 16, 8)
    s = c.admit()
    for _ in range(16):
        c.reserve(s, 1)
        c.commit(s, 1)
    assert len(c.block_table(s, 0)) == 1 and c.cached(s) == 16 and c.free_pages(0) == 7
    c.release(s)
    assert c.free_pages(0) == 8
    c.check()


def test_layers_are_grouped_by_need():
    c = make([CHUNK32, CHUNK32, CHUNK32, FULL])            # tiny A: three rotating layers, one NoPE
    assert c.n_groups() == 2 and c.groups[0].cache_ids == [0, 1, 2] and c.groups[1].cache_ids == [3]
    assert c.group_of(3) == 1
    other_heads = make([FULL, CacheNeed(kv=KVNeed(4, 16, "full")), None])
    assert other_heads.n_groups() == 2                      # other head count: pages of their own


def test_pages_grow_with_tokens_and_tables_are_per_group():
    c = make([CHUNK32, FULL], 16, 8)
    s = c.admit()
    c.reserve(s, 40)
    assert c.block_table(s, 0) == [0, 1, 2] == c.block_table(s, 1)
    assert c.free_pages(0) == 5 and c.free_pages(1) == 5
    c.commit(s, 40)
    # the next query sits at 40, chunk [32,64): blocks 0 and 1 of the chunked group are behind it
    assert c.block_table(s, 0) == [-1, -1, 2] and c.block_table(s, 1) == [0, 1, 2]
    assert c.free_pages(0) == 7 and c.free_pages(1) == 5
    c.check()


def test_a_portion_across_a_chunk_border_keeps_its_pages_until_the_step_is_over():
    c = make([CHUNK32], 16, 8)
    s = c.admit()
    c.reserve(s, 30); c.commit(s, 30)
    c.reserve(s, 10)                                        # positions 30..39 straddle the border at 32
    assert c.block_table(s, 0) == [0, 1, 2]                 # nothing given back before the commit
    m = np.zeros(10, dtype=np.int32)
    c.fill_step([s], [30], [10], 0, m, np.zeros((1, 4), dtype=np.int32))
    assert m.tolist() == [16 + 14, 16 + 15] + [32 + i for i in range(8)]
    c.commit(s, 10)
    assert c.block_table(s, 0) == [-1, -1, 2]


def test_window_gives_back_what_no_later_query_reads():
    c = make([WIN20], 16, 8)
    s = c.admit()
    c.reserve(s, 50); c.commit(s, 50)                       # next query at 50 reads from 31: block 0 is behind
    assert c.block_table(s, 0) == [-1, 1, 2, 3]
    c.reserve(s, 2); c.commit(s, 2)                         # next at 52 reads from 33: block 1 too
    assert c.block_table(s, 0) == [-1, -1, 2, 3]


def test_pages_that_are_given_back_are_handed_out_next():
    c = make([FULL], 16, 4)
    a = c.admit(); c.reserve(a, 32); c.commit(a, 32)
    b = c.admit(); c.reserve(b, 16); c.commit(b, 16)
    assert c.block_table(a, 0) == [0, 1] and c.block_table(b, 0) == [2]
    c.release(a)
    d = c.admit(); c.reserve(d, 40)
    assert c.block_table(d, 0) == [0, 1, 3]                 # a's pages first, in its order
    c.check()


def test_a_step_gets_all_its_pages_or_none():
    c = make([CHUNK32, FULL], 16, 5)
    a, b, d = c.admit(), c.admit(), c.admit()
    c.reserve_all([(a, 20), (b, 16)])                       # 2 + 1 pages of either group
    assert c.free_pages(0) == 2 and c.free_pages(1) == 2
    with pytest.raises(OutOfPages):                         # a: none more, b: one more, d: two: three in all
        c.reserve_all([(a, 30), (b, 17), (d, 20)])
    assert c.free_pages(0) == 2 and len(c.block_table(b, 0)) == 1 and c.block_table(d, 0) == []
    c.reserve_all([(a, 30), (b, 17), (d, 16)])              # one for b, one for d
    assert c.free_pages(0) == 0 and c.free_pages(1) == 0
    with pytest.raises(CacheError):
        c.reserve_all([(a, 1), (a, 1)])
    c.check()


def test_running_out_changes_nothing():
    c = make([CHUNK32, FULL], 16, 3)
    s = c.admit()
    c.reserve(s, 48)
    t = c.admit()
    assert not c.can_reserve(t, 1)
    with pytest.raises(OutOfPages):
        c.reserve(t, 1)
    assert c.block_table(t, 0) == [] and c.free_pages(0) == 0 and c.free_pages(1) == 0
    c.commit(s, 48)                                         # chunk roll-off frees the chunked group only
    assert c.free_pages(0) == 2 and c.free_pages(1) == 0
    assert not c.can_reserve(t, 1)                          # the full group is still short
    c.check()


def test_slots_and_errors():
    c = make([FULL], 16, 4, max_requests=2)
    a, b = c.admit(), c.admit()
    assert {a, b} == {0, 1} and c.free_slots() == 0
    with pytest.raises(CacheError, match="slots"):
        c.admit()
    c.release(a)
    with pytest.raises(CacheError):
        c.release(a)                                        # freed twice
    with pytest.raises(CacheError):
        c.commit(b, 1)                                      # more than was reserved
    with pytest.raises(CacheError):
        c.reserve(a, 1)                                     # not live
    assert c.admit() == a


def test_peak_pages():
    c = make([CHUNK32, FULL], 16, 8)
    assert c.peak_pages(100, 1000, 1) == 7                  # full: every page
    assert c.peak_pages(100, 8, 0) == 3                     # chunk 32 in portions of 8: a chunk plus a page
    assert c.peak_pages(100, 1000, 0) == 7                  # one portion needs them all at once


def test_state_slots_are_zeroed_on_admission():
    c = PagedCache([CacheNeed(state=StateNeed((3, 2))), FULL], 16, 4, 2, torch.float32, torch.device("cpu"))
    assert c.states[0].shape == (2, 3, 2) and 1 not in c.states
    s = c.admit()
    c.states[0][s] += 5.0
    c.release(s)
    assert c.admit() == s and float(c.states[0][s].abs().sum()) == 0.0


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_keep_the_books(seed):
    rnd = random.Random(seed)
    ps = rnd.choice([4, 16])
    needs = [CHUNK32, FULL, WIN20, CHUNK32]
    c = make(needs, ps, pages=rnd.choice([6, 12, 40]), max_requests=4)
    live = {}
    spans = {0: ("chunk", 32), 1: ("full", 0), 2: ("window", 20)}
    for _ in range(400):
        op = rnd.random()
        if op < 0.2 and c.free_slots():
            live[c.admit()] = 0
        elif op < 0.3 and live:
            s = rnd.choice(list(live))
            c.release(s); del live[s]
        elif live:
            s = rnd.choice(list(live))
            n = rnd.choice([1, 1, 2, 5, 17, 40])
            if c.can_reserve(s, n):
                before = [c.free_pages(g) for g in range(3)]
                c.reserve(s, n)
                c.commit(s, n)
                live[s] += n
                # what is held is exactly what a later query can read
                for g, (kind, span) in spans.items():
                    tab = c.block_table(s, g)
                    first = {"full": 0, "chunk": (live[s] // 32) * 32, "window": max(live[s] - 20 + 1, 0)}[kind]
                    for b, page in enumerate(tab):
                        behind = (b + 1) * ps <= first
                        assert (page < 0) == behind, (kind, live[s], tab)
                    assert len(tab) == -(-live[s] // ps)
            else:
                free = [c.free_pages(g) for g in range(3)]
                with pytest.raises(OutOfPages):
                    c.reserve(s, n)
                assert free == [c.free_pages(g) for g in range(3)]
        c.check()                                           # no page lost, held twice or free twice
        assert sum(len([p for p in c.block_table(s, 1) if p >= 0]) for s in live) + c.free_pages(1) == c.total_pages(1)
    for s in list(live):
        c.release(s)
    assert all(c.free_pages(g) == c.total_pages(g) for g in range(3))


def test_slots_handed_out_are_reported_once_whoever_admitted_them():
    # the native scheduler admits behind the Python object's back; the state rows of every slot
    # handed out are cleared before the next step, so a request never meets its predecessor's state
    from spite_amd.engine.scheduler import Scheduler
    need = CacheNeed(kv=KVNeed(1, 16, "full"), state=StateNeed((3,), torch.float32))
    c = PagedCache([need], 16, 8, 3, torch.float32, torch.device("cpu"))
    c.states[0][:] = 7.0
    s = c.admit()
    assert c.states[0][s].abs().sum() == 0 and c.states[0].abs().sum() == 2 * 3 * 7.0
    assert c.zero_fresh() == []
    c.states[0][:] = 7.0
    sched = Scheduler(c, 32, 1000)
    sched.submit([1, 2, 3], 4)
    sched.submit([4, 5], 4)
    batch = sched.schedule()                                # admits two slots natively
    assert sorted(b.slot for b in batch) == [1, 2]
    assert c.states[0][1:].abs().sum() > 0                  # nothing cleared yet
    assert c.zero_fresh() == [1, 2]
    assert c.states[0][1:].abs().sum() == 0 and c.states[0][s].abs().sum() == 21.0
    assert c.zero_fresh() == []
    # released and admitted again between two steps: reported, once
    c.release(s)
    assert c.admit() == s and c.states[0][s].abs().sum() == 0


def test_a_storm_of_admissions_clears_no_running_request():
    # many admissions and releases between two steps: every slot that changed hands is reported
    # once, and the state of a request that kept running meanwhile is not touched
    need = CacheNeed(kv=KVNeed(1, 16, "full"), state=StateNeed((3,), torch.float32))
    c = PagedCache([need], 16, 8, 3, torch.float32, torch.device("cpu"))
    runner = c.admit()
    assert c.zero_fresh() == []
    c.states[0][runner] = 5.0
    lib, h = c._lib, c._h
    for _ in range(200):                                     # behind the Python object's back, as a scheduler would
        s = lib.spc_admit(h)
        assert s >= 0 and s != runner
        lib.spc_release(h, s)
    s = lib.spc_admit(h)
    c.states[0][s] = 9.0
    got = c.zero_fresh()
    assert s in got and runner not in got and len(got) == len(set(got)) <= 2
    assert c.states[0][runner].tolist() == [5.0] * 3 and c.states[0][s].abs().sum() == 0


def test_a_chunked_group_gets_no_more_pages_than_its_requests_can_hold():
    needs = [CacheNeed(kv=KVNeed(8, 128, "chunk", 8192)), CacheNeed(kv=KVNeed(8, 128, "full")),
             CacheNeed(kv=KVNeed(8, 128, "window", 100))]
    c = PagedCache(needs, 64, 8 * 32768 // 64, 8, torch.bfloat16, torch.device("cpu"), allocate=False, portion=2048)
    # a chunk of 8,192 and a portion of 2,048 are 160 pages of 64; the whole context stays with the full group
    assert [c.total_pages(g) for g in range(3)] == [8 * 160, 8 * 512, 8 * c.peak_pages(32768, 2048, 2)]
    assert c.peak_pages(32768, 2048, 2) == (100 + 2048 - 2) // 64 + 2
    # eight requests of 30,000 tokens in portions of 2,048 never run out in the chunked group
    slots = [c.admit() for _ in range(8)]
    for at in range(0, 30000, 2048):
        n = min(2048, 30000 - at)
        for s in slots:
            c.reserve(s, n)
        for s in slots:
            c.commit(s, n)
    c.check()
    # small pools are left as they are
    small = PagedCache(needs[:2], 16, 8, 4, torch.float32, torch.device("cpu"), allocate=False, portion=2048)
    assert [small.total_pages(g) for g in range(2)] == [8, 8]


def test_keys_and_values_of_widths_of_their_own():
    # a mixer whose values are wider than its keys: the pool's halves are sized apart, and such a
    # need shares no group with one of equal widths
    needs = [CacheNeed(kv=KVNeed(2, 8, "full", 0, v_head_dim=24)), CacheNeed(kv=KVNeed(2, 8, "full")),
             CacheNeed(kv=KVNeed(2, 8, "full", 0, v_head_dim=24))]
    c = PagedCache(needs, 4, 6, 2, torch.float32, torch.device("cpu"))
    assert c.n_groups() == 2 and c.group_of(0) == c.group_of(2) != c.group_of(1)
    k, v = c.layer_pages(2)
    assert tuple(k.shape) == (6, 2, 4, 8) and tuple(v.shape) == (6, 2, 24, 4)
    k1, v1 = c.layer_pages(1)
    assert tuple(k1.shape) == (6, 2, 4, 8) and tuple(v1.shape) == (6, 2, 8, 4)
    assert not c.kv_tiled(0)


def test_the_visibility_rules_have_one_definition():
    """The names and codes of the rules that say which keys a query reads come from one header;
    the cache manager (native) frees exactly what that header's rule no longer reads."""
    from spite_amd.csrc import build, hipops, hostlib
    from spite_amd.cache import paged
    codes = build.visibility_codes()
    assert codes == {"full": 0, "chunk": 1, "window": 2} and hipops.VIS == codes and paged._KINDS == codes
    lib = hostlib.lib()
    for kind, span, n, first in (("full", 0, 37, 0), ("chunk", 8, 37, 32), ("window", 8, 37, 30), ("window", 8, 5, 0)):
        h = lib.spc_create(4, 1, 1, hostlib.int_array([codes[kind]]), hostlib.int_array([span]), hostlib.int_array([32]))
        s = lib.spc_admit(h)
        assert lib.spc_reserve(h, s, n) == 0 and lib.spc_commit(h, s, n) == 0
        n_tab = lib.spc_table_len(h, s, 0)
        tab = hostlib.int_array([0] * n_tab)
        lib.spc_table(h, s, 0, tab, n_tab)
        held = [i for i in range(n_tab) if tab[i] >= 0]
        # the next query (position n) reads from `first`: pages wholly below it are gone
        assert held == list(range(first // 4, -(-n // 4))), (kind, span, held)
        lib.spc_destroy(h)
