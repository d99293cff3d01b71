"""Faults planted in the engine, to show that the engine-level checks would see them, and that
what a request does not own cannot reach it.

* Every page that no live request holds is overwritten with NaN after every step (keys and
  values, every layer).  Pages are handed out again from that pool, so a request's newest page
  holds NaN behind its last position.  The logits must stay finite and equal to a clean run's
  bit for bit: a probability of zero must not meet a value that is not finite.
* A block-table entry is pointed at a page that the request does not hold (full of large
  values), or is taken away: the logits move by far more than the tolerance of the replay tests,
  or are NaN (the kernels poison what they are asked to read from a page that is not there).
"""
import numpy as np
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu

# "Cw": a window of 100 keys over pages of 32: the first visible key's page has an odd index at
# times, so that a block of 64 keys begins on a page that the request has already given back
CASES = [("A", "float32", 16), ("B", "float32", 8), ("C", "bfloat16", 32), ("C", "float32", 32),
         ("Cw", "bfloat16", 32), ("Bw", "float32", 8)]


def steps_for(cfg):
    V = cfg["vocab_size"]
    a, b, c = (H.random_tokens(V, n, 10 + i) for i, n in enumerate((150, 90, 41)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [69]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[70:72], "want": [0, 1]},
                                     {"id": "b", "tokens": b[:33], "want": [32]}], "end": []}]
    at_a, at_b = 72, 33
    for j in range(40):                  # a decodes and ends; c then takes over its pages; b runs all the way
        entries, ended = [], []
        if j < 20:
            entries.append({"id": "a", "tokens": [a[at_a]], "want": [0]})
            at_a += 1
            if j == 19:
                ended.append("a")
        n = 7 if at_b < 75 else 1
        if at_b < len(b):
            entries.append({"id": "b", "tokens": b[at_b:at_b + n], "want": [n - 1]})
            at_b += n
        if j == 20:
            entries.append({"id": "c", "tokens": c[:30], "want": [29]})
        elif 20 < j <= 31:
            entries.append({"id": "c", "tokens": [c[30 + j - 21]], "want": [0]})
            if j == 31:
                ended.append("c")
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def pool_tokens(page):
    up = lambda n: -(-n // page) * page
    return up(92) + up(90) + page          # a and b together, and a page to spare; c lives on a's pages


def held_pages(eng, g):
    held = set()
    for s in range(eng.cache.max_requests):
        if eng.cache.live(s):
            held |= {p for p in eng.cache.block_table(s, g) if p >= 0}
    return held


def poison_what_nobody_holds(eng, value=float("nan")):
    for g, group in enumerate(eng.cache.groups):
        free = sorted(set(range(group.n_pages)) - held_pages(eng, g))
        if free:
            for half in group.halves():
                half[:, torch.tensor(free, device=half.device)] = value


def run(eng, steps, after_step=None):
    from spite_amd.engine.engine import StepEntry
    slots, out = {}, {}
    for rec in steps:
        entries = []
        for e in rec["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = eng.admit()
            entries.append(StepEntry(slots[e["id"]], e["tokens"], e["want"]))
        out[rec["step"]] = eng.step(entries).cpu().numpy().copy()
        for rid in rec["end"]:
            eng.release(slots.pop(rid))
        if after_step is not None:
            after_step(eng)
    return out


@pytest.mark.parametrize("name,dtype,page", CASES, ids=[f"{n}-{d}" for n, d, _ in CASES])
def test_pages_that_nobody_holds_cannot_reach_a_request(name, dtype, page, tmp_path):
    from spite_amd.engine.engine import Engine
    cfg = H.CONFIGS[name]
    d = str(tmp_path / "m")
    H.make_model(d, cfg, seed=9, dtype=dtype)
    steps = steps_for(cfg)
    make = lambda: Engine(d, dtype=dtype, page_size=page, cache_tokens=pool_tokens(page), max_requests=3, graphs=False)
    clean = run(make(), steps)
    dirty_engine = make()
    poison_what_nobody_holds(dirty_engine)
    dirty = run(dirty_engine, steps, after_step=poison_what_nobody_holds)
    # pages were used again: fewer pages than the three requests' positions need together
    assert pool_tokens(page) < sum(-(-n // page) * page for n in (92, 90, 41))
    for k in clean:
        assert np.isfinite(dirty[k]).all(), f"step {k}: a value that nobody holds reached the logits"
        assert np.array_equal(clean[k], dirty[k]), f"step {k}"


@pytest.mark.parametrize("name,dtype,page", CASES, ids=[f"{n}-{d}" for n, d, _ in CASES])
def test_a_wrong_block_table_entry_shows(name, dtype, page, tmp_path):
    from spite_amd.engine.engine import Engine
    cfg = H.CONFIGS[name]
    d = str(tmp_path / "m")
    H.make_model(d, cfg, seed=9, dtype=dtype)
    steps = steps_for(cfg)[:12]
    make = lambda: Engine(d, dtype=dtype, page_size=page, cache_tokens=pool_tokens(page), max_requests=3, graphs=False)
    clean = run(make(), steps)
    scale = max(float(np.abs(v).max()) for v in clean.values())
    tol = 2e-5 if dtype == "float32" else 0.04 * scale

    def tamper(eng, how):
        original = eng.cache.fill_step

        def fill_step(slots, starts, counts, g, slot_map_out, table_out):
            original(slots, starts, counts, g, slot_map_out, table_out)
            if eng.steps_run == 8 and eng.cache.groups[g].key[2] == "full":
                row = table_out[0]
                live = [i for i, p in enumerate(row) if p >= 0]
                if how == "other page":
                    free = sorted(set(range(eng.cache.groups[g].n_pages)) - held_pages(eng, g))
                    row[live[0]] = free[-1]
                else:
                    row[live[0]] = -1
        eng.cache.fill_step = fill_step

    for how in ("other page", "no page"):
        eng = make()
        poison_what_nobody_holds(eng, 3.0)
        tamper(eng, how)
        got = run(eng, steps, after_step=lambda e: poison_what_nobody_holds(e, 3.0))
        for k in clean:
            if k < 8:                           # the steps before it are untouched
                assert np.array_equal(clean[k], got[k]), (how, k)
        diff = np.abs(got[8][0].astype(np.float64) - clean[8][0])
        if how == "no page":
            assert np.isnan(got[8][0]).all(), "a page that is not there must poison the request that asks for it"
            assert np.isfinite(got[8][1:]).all(), "and only that request"
        else:
            assert np.isnan(diff).any() or diff.max() > 5 * tol, (how, diff.max(), tol)
