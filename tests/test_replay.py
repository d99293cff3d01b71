"""Replay on the GPU: the same requests whole, with the last 32 tokens one by one, in
portions of changing size, and mixed with other requests on a pool so small that pages are
used again - in 32-bit and in bfloat16, each compared with the plain implementation and with
each other.  The logits at a position must not depend on how the tokens were cut into
steps, on what else was in the batch, or on which pages were used."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

# fp32: the engine against the float64 plain implementation; logits are O(1).
TOL_F32 = 2e-5
# fp32, one schedule against another: the kernels' sums do not depend on the batch.
TOL_F32_SCHEDULES = 2e-6
# bfloat16: relative to the largest logit of the request set.  Activations are rounded to 8
# bits of mantissa (unit roundoff 2^-9) some six times a layer; over the tiny models' layers
# that is about one percent of the scale.  A wrong mask, page or expert moves the planted
# models' logits by ten percent and more (see test_faults_are_visible).
TOL_BF16_REL = 0.04
# bfloat16 only: the router's logits come from the same hidden states and carry the same
# relative error as the output logits.  Where the plain implementation's best two router
# logits of a token lie within that accepted error (this fraction of the size of the layer's
# router logits, their root mean square), the experts are tied at bfloat16's precision; the plain
# implementation then follows the engine's choice, and the logits must agree within the
# tolerance under that choice.  A choice further off is not followed and shows as a fault.
HINT_REL = TOL_BF16_REL

REQUESTS = {
    "A": {"a0": 5 + 16, "a1": 23 + 16, "a2": 40 + 16, "a3": 131},
    "B": {"b0": 1 + 16, "b1": 7 + 16, "b2": 16 + 16, "b3": 33 + 16, "b4": 70 + 16},
    "C": {"c0": 5 + 16, "c1": 70, "c2": 150, "c3": 300},
}
REQUESTS.update({"Bw": REQUESTS["B"], "Cw": REQUESTS["C"], "Cm": REQUESTS["C"]})
PAGE = {"A": 16, "B": 8, "C": 32, "Bw": 8, "Cw": 32, "Cm": 32}


class Case:
    def __init__(self, name, dtype, tmp):
        from spite_amd.engine.engine import Engine
        self.name, self.dtype, self.cfg = name, dtype, H.CONFIGS[name]
        self.dir = str(tmp / f"{name}_{dtype}")
        self.weights = H.make_model(self.dir, self.cfg, seed=7, dtype=dtype, keep_wide=H.KEEP_WIDE.get(name, ()))
        self.reqs = {rid: H.random_tokens(self.cfg["vocab_size"], n, 100 + i)
                     for i, (rid, n) in enumerate(REQUESTS[name].items())}
        self.plain = H.plain_logits(self.cfg, self.weights, self.reqs)
        self.scale = max(float(np.abs(v).max()) for v in self.plain.values())
        self.tol = TOL_F32 if dtype == "float32" else TOL_BF16_REL * self.scale
        self.results = {}
        self.Engine = Engine
        # a pool for one request at a time, whole
        self.pool = max(256, -(-max(len(t) for t in self.reqs.values()) // PAGE[name]) * PAGE[name])

    def engine(self, cache_tokens, page_size=None, max_requests=4):
        return self.Engine(self.dir, dtype=self.dtype, page_size=page_size or PAGE[self.name],
                           cache_tokens=cache_tokens, max_requests=max_requests, max_batch_tokens=4096)

    def replay(self, steps, cache_tokens, take=None, **kw):
        eng = self.engine(cache_tokens, **kw)
        routing = {}
        out = H.run_trace_inprocess(eng, steps, routing, take=take)
        for g in range(eng.cache.n_groups()):
            assert eng.cache.free_pages(g) == eng.cache.total_pages(g)
        return H.collect(steps, out, self.cfg["vocab_size"]), H.routing_hints(self.cfg, steps, routing)

    def reference(self, reqs, hints):
        """The plain implementation's logits; in bfloat16 with the engine's expert wherever
        the plain implementation's own choice was a near tie."""
        if self.dtype == "float32":
            return {k: v for k, v in self.plain.items() if k[0] in reqs} if all(r in self.reqs for r in reqs) \
                else H.plain_logits(self.cfg, self.weights, reqs)
        taken, differ = [], []
        ref = H.plain_logits(self.cfg, self.weights, reqs, hints, HINT_REL, taken, differ)
        n_tok = sum(len(t) for t in reqs.values()) * len(H.moe_layers(self.cfg))
        print(f"[{self.name} {self.dtype}] routing: {len(taken)} near ties followed, {len(differ)} choices "
              f"differ beyond a tie {differ[:4]} (of {n_tok})")
        assert len(taken) <= max(3, 0.03 * n_tok), f"{len(taken)} of {n_tok} routing choices were near ties"
        return ref


@pytest.fixture(scope="module", params=[("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16"), ("C", "bfloat16"),
                                        ("Bw", "float32"), ("Bw", "bfloat16"), ("Cw", "bfloat16"), ("Cm", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def case(request, tmp_path_factory):
    return Case(*request.param, tmp_path_factory.mktemp("replay"))


def check(case, result, label, reqs=None):
    rows, hints = result
    ref = case.reference(reqs or case.reqs, hints)
    d, where = H.max_diff(rows, ref)
    print(f"[{case.name} {case.dtype}] {label}: max|diff| vs plain {d:.3e} at {where} (tol {case.tol:.3e}, scale {case.scale:.2f})")
    assert d <= case.tol, f"{label}: {d} at {where}"
    case.results[label] = rows


def test_whole(case):
    check(case, case.replay(H.schedule_whole(case.reqs), case.pool), "whole")


def test_last_32_one_by_one(case):
    check(case, case.replay(H.schedule_tail_one_by_one(case.reqs), case.pool), "tail")


def test_portions_of_changing_size(case):
    steps = H.schedule_portions(case.reqs)
    assert min(len(e["tokens"]) for s in steps for e in s["entries"]) <= 2
    check(case, case.replay(steps, case.pool), "portions")


def test_mixed_with_pages_used_again(case):
    steps = H.schedule_mixed(case.reqs, seed=3)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(e["tokens"]) > 1 for s in steps for e in s["entries"] if len(s["entries"]) > 1)
    # the pool: what the four largest requests hold, each rounded up to its pages
    ps = PAGE[case.name]
    sizes = sorted((-(-len(t) // ps) * ps for t in case.reqs.values()), reverse=True)
    eng = case.engine(sum(sizes[:4]))
    seen_pages, reused = set(), False
    from spite_amd.engine.engine import StepEntry
    slots, out, routing = {}, {}, {}
    for rec in steps:
        entries = []
        for e in rec["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = eng.admit()
            entries.append(StepEntry(slots[e["id"]], e["tokens"], e["want"]))
        trace = {}
        out[rec["step"]] = eng.step(entries, trace=trace).cpu().numpy().copy()
        routing[rec["step"]] = [t.cpu().numpy() for t in trace.get("moe_experts", [])]
        for s in slots.values():
            for g in range(eng.cache.n_groups()):
                for b, p in enumerate(eng.cache.block_table(s, g)):
                    if p >= 0:
                        key = (g, p)
                        owner = (s, b)
                        reused |= any(k == key and o != owner for k, o in seen_pages)
                        seen_pages.add((key, owner))
        for rid in rec["end"]:
            eng.release(slots.pop(rid))
        eng.cache.check()
    assert reused, "the pool was large enough that no page was handed out twice"
    check(case, (H.collect(steps, out, case.cfg["vocab_size"]), H.routing_hints(case.cfg, steps, routing)), "mixed")


def test_decoded_tokens_lead_a_mixed_step(case, monkeypatch):
    """The scheduler's own order: one decoded token of each running request first, portions of
    prompts behind them.  Where the MFMA attention kernels run, the mixer gives the leading
    tokens to the decode kernel and the portions to the prefill kernel."""
    from spite_amd.csrc import hipops
    ids = list(case.reqs)[-3:]
    a, b, c = (case.reqs[i] for i in ids)
    ka, kb = len(a) - 3, len(b) - 3
    cut = [0, len(c) * 2 // 5, len(c) * 4 // 5, len(c)]
    steps = [{"step": 0, "entries": [{"id": ids[0], "tokens": a[:ka], "want": list(range(ka))}], "end": []},
             {"step": 1, "entries": [{"id": ids[1], "tokens": b[:kb], "want": list(range(kb))}], "end": []}]
    for j in range(3):
        steps.append({"step": 2 + j, "entries": [
            {"id": ids[0], "tokens": [a[ka + j]], "want": [0]}, {"id": ids[1], "tokens": [b[kb + j]], "want": [0]},
            {"id": ids[2], "tokens": c[cut[j]:cut[j + 1]], "want": list(range(cut[j + 1] - cut[j]))}],
            "end": ids if j == 2 else []})
    calls = []
    real = hipops.attn_decode

    def counted(q, k, v, out, ws, pos, seq, bt, T, *args, **kw):
        calls.append((T, pos.numel()))
        return real(q, k, v, out, ws, pos, seq, bt, T, *args, **kw)
    monkeypatch.setattr(hipops, "attn_decode", counted)
    reqs = {i: case.reqs[i] for i in ids}
    ps = PAGE[case.name]
    check(case, case.replay(steps, sum(-(-len(t) // ps) * ps for t in reqs.values())), "decodes first", reqs)
    if case.dtype == "bfloat16" and case.cfg["head_dim"] in (64, 128):
        assert calls and all(T == 2 and n > 2 for T, n in calls), calls[:4]
    else:
        assert not calls


def test_schedules_agree_with_each_other(case):
    need = ["whole", "tail", "portions", "mixed"]
    if any(k not in case.results for k in need):
        pytest.skip("an earlier replay failed")
    if case.dtype == "float32":
        for k in need[1:]:
            d, where = H.max_diff(case.results[k], case.results["whole"])
            print(f"[{case.name} {case.dtype}] {k} vs whole: {d:.3e}")
            assert d <= TOL_F32_SCHEDULES, f"{k} differs from whole by {d} at {where}"
        return
    # In bfloat16 a near tie of two experts may fall differently in two schedules (the decode and
    # the prefill kernels group their sums differently), and a token with another expert is
    # another computation.  So the schedules are run again with the experts that the whole
    # replay took: what is left is rounding, and the schedules have to agree to it.
    ps = PAGE[case.name]
    pool = sum(sorted((-(-len(t) // ps) * ps for t in case.reqs.values()), reverse=True)[:4])
    whole_steps = H.schedule_whole(case.reqs)
    whole, hints = case.replay(whole_steps, case.pool)
    schedules = {"tail": H.schedule_tail_one_by_one(case.reqs), "portions": H.schedule_portions(case.reqs),
                 "mixed": H.schedule_mixed(case.reqs, seed=3)}
    for k, steps in schedules.items():
        rows, _ = case.replay(steps, pool, take=H.experts_to_take(case.cfg, steps, hints))
        d, where = H.max_diff(rows, whole)
        print(f"[{case.name} {case.dtype}] {k} with the whole replay's experts vs whole: {d:.3e} (tol {case.tol:.3e})")
        assert d <= case.tol, f"{k} differs from whole by {d} at {where}"


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_other_mixed_schedules_agree_with_whole(case, seed):
    """More ways of cutting and mixing the same requests, also with portions of 31 and 64 tokens
    (a page's edge, a chunk's edge, several pages in one portion), against the whole replay;
    in bfloat16 with the whole replay's experts."""
    if "whole" not in case.results:
        pytest.skip("the whole replay failed")
    ps = PAGE[case.name]
    pool = sum(sorted((-(-len(t) // ps) * ps for t in case.reqs.values()), reverse=True)[:4])
    steps = H.schedule_mixed(case.reqs, seed=seed, portion_sizes=(2, 3, 5, 8, 13, 31, 64))
    take = None
    if case.dtype != "float32":
        whole_steps = H.schedule_whole(case.reqs)
        if not hasattr(case, "whole_hints"):
            case.whole_rows, case.whole_hints = case.replay(whole_steps, case.pool)
        take = H.experts_to_take(case.cfg, steps, case.whole_hints)
    rows, _ = case.replay(steps, pool, take=take)
    want = case.results["whole"] if case.dtype == "float32" else case.whole_rows
    d, where = H.max_diff(rows, want)
    tol = TOL_F32_SCHEDULES if case.dtype == "float32" else case.tol
    print(f"[{case.name} {case.dtype}] mixed schedule {seed} vs whole: {d:.3e} (tol {tol:.3e})")
    assert d <= tol, f"schedule {seed} differs from whole by {d} at {where}"


def test_first_tokens_of_a_sequence(case):
    # one-token and two-token requests, and position 0 of every request
    first = case.reqs[next(iter(case.reqs))]
    reqs = {"p1": first[:1], "p2": first[:2]}
    check(case, case.replay(H.schedule_whole(reqs), 64), "first tokens", reqs)


def test_long_decoding(case):
    # 8 tokens of prompt, then 150 decoded one by one: chunk borders, temperature steps and
    # many pages of the full group are crossed token by token
    reqs = {"long": H.random_tokens(case.cfg["vocab_size"], 158, 55)}
    check(case, case.replay(H.schedule_tail_one_by_one(reqs, tail=150), 160), "long decode", reqs)


def test_the_step_has_no_context_limit(tmp_path):
    """``max_position_embeddings`` bounds what generation is asked for, not what a step runs:
    a replay that goes past it gives the plain implementation's logits."""
    from spite_amd.engine.engine import Engine
    cfg = dict(H.CONFIGS["A"], max_position_embeddings=32)
    folder = str(tmp_path / "short_limit")
    weights = H.make_model(folder, cfg, seed=9, dtype="float32")
    reqs = {"x": H.random_tokens(cfg["vocab_size"], 75, 3)}
    steps = H.schedule_portions(reqs)
    eng = Engine(folder, dtype="float32", page_size=16, cache_tokens=128, max_requests=2)
    rows = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab_size"])
    d, where = H.max_diff(rows, H.plain_logits(cfg, weights, reqs))
    assert d <= TOL_F32, (d, where)


def test_trace_run_program(case):
    """The program itself, as a user runs it: page size 64, the pool given by --max-tokens."""
    reqs = dict(list(case.reqs.items())[:3])
    steps = H.schedule_mixed(reqs, seed=1, max_live=2)
    sizes = sorted((-(-len(t) // 64) * 64 for t in reqs.values()), reverse=True)
    routing = {}
    out = H.run_trace_program(case.dir, case.dtype, steps, sum(sizes[:2]), routing=routing)
    check(case, (H.collect(steps, out, case.cfg["vocab_size"]), H.routing_hints(case.cfg, steps, routing)),
          "trace_run", reqs)


def test_faults_are_visible(case):
    """The tolerance tells a right engine from a wrong one: the plain implementation with
    the reference's sliding window in place of chunks, or with one expert swapped, differs
    from the right logits by far more than the tolerance."""
    import plain_llama4 as plain
    rid = {"A": "a3", "B": "b4", "C": "c3"}[case.name[0]]
    toks = case.reqs[rid]
    right = np.stack([case.plain[(rid, i)] for i in range(len(toks))])
    other = "chunk" if case.cfg.get("attention_local_kind") == "window" else "window"
    window = plain.forward(case.cfg, case.weights, toks, visibility=other).numpy()
    assert np.abs(window - right).max() > 3 * case.tol
    w2 = dict(case.weights)
    moe_layer = 1
    k = f"model.layers.{moe_layer}.feed_forward.experts.down_proj"
    w2[k] = case.weights[k].roll(1, dims=0)
    swapped = plain.forward(case.cfg, w2, toks).numpy()
    assert np.abs(swapped - right).max() > 3 * case.tol
