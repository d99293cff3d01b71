"""Long context through the engine's step function with the real chunk size and temperature
constants (attention_chunk_size 8192, floor_scale 8192): one request of 17,000 tokens fed in
portions of 2,048, then tokens one by one, beside a short request that decodes meanwhile, in
32-bit and in bfloat16, against the plain implementation at a few hundred positions on either
side of 8,192 and 16,384.  The model is narrow (three layers: rotating and chunked, without
position and full, rotating and chunked) so that the plain implementation takes seconds.

Random weights would hide a lost key among 17,000.  Here the one kv head's key projection is
head 0's query projection, so a token scores high against every earlier copy of itself: some
thirty keys anywhere in the context carry most of a query's attention, and a wrong chunk edge,
a missing page or a wrong temperature moves the logits far beyond the tolerance
(``test_a_wrong_chunk_or_temperature_is_visible``)."""
import numpy as np
import pytest
import torch

import helpers as H
import plain_llama4 as plain

pytestmark = pytest.mark.gpu

CHUNK, PORTION, PAGE = 8192, 2048, 64
N_LONG, N_DECODE = 17000, 8
CFG = dict(
    architectures=["Llama4ForCausalLM"], num_hidden_layers=3, hidden_size=128, num_attention_heads=2,
    num_key_value_heads=1, head_dim=64, rms_norm_eps=1e-5, num_local_experts=4, num_experts_per_tok=1,
    intermediate_size=128, intermediate_size_mlp=256, interleave_moe_layer_step=1, vocab_size=512,
    rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=16.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    attention_chunk_size=CHUNK, no_rope_layers=[1, 0, 1], use_qk_norm=True, attn_temperature_tuning=True,
    floor_scale=8192, attn_scale=0.1, tie_word_embeddings=False, torch_dtype="float32")
# 32-bit: the engine against the float64 plain implementation, whose rotation angles are
# formed in 32-bit as the reference forms them (at 17,000 an angle in 32-bit is a thousandth of
# a radian off, which alone moves these logits by 1e-4); logits are O(1)
TOL_F32 = 3e-5
TOL_BF16_REL = 0.04


def planted(seed):
    t = H.planted_tensors(CFG, seed)
    hd = CFG["head_dim"]
    for L in range(CFG["num_hidden_layers"]):
        p = f"model.layers.{L}.self_attn."
        t[p + "k_proj.weight"] = t[p + "q_proj.weight"][:hd].clone()      # the kv head looks like query head 0
    return t


def wanted_positions():
    rng = np.random.RandomState(5)
    edges = [0, 1, 63, 64, PORTION - 1, PORTION, CHUNK - 65, CHUNK - 64, CHUNK - 2, CHUNK - 1, CHUNK, CHUNK + 1,
             CHUNK + 63, CHUNK + 64, CHUNK + PORTION - 1, CHUNK + PORTION, 2 * CHUNK - 2, 2 * CHUNK - 1, 2 * CHUNK,
             2 * CHUNK + 1, 2 * CHUNK + 64, N_LONG - 1]
    spread = rng.choice(N_LONG, 230, replace=False).tolist()
    return sorted(set(edges + spread))


def schedule(long_toks, short_toks):
    """The long request in portions of 2,048 and then token by token; the short one whole in the
    first step and then one token a step in front of the long one's portions (mixed steps)."""
    want = set(wanted_positions())
    steps, at, fed_short = [], 0, 0
    n_prompt_short = len(short_toks) - 12
    while at < len(long_toks):
        n = min(PORTION, N_LONG - at) if at < N_LONG else 1
        entries = []
        if fed_short == 0:
            entries.append({"id": "short", "tokens": short_toks[:n_prompt_short], "want": [n_prompt_short - 1]})
            fed_short = n_prompt_short
        elif fed_short < len(short_toks):
            entries.append({"id": "short", "tokens": [short_toks[fed_short]], "want": [0]})
            fed_short += 1
        w = [p - at for p in range(at, at + n) if p in want or p >= N_LONG]
        entries.append({"id": "long", "tokens": long_toks[at:at + n], "want": w})
        at += n
        ended = [rid for rid, done in (("short", fed_short == len(short_toks)), ("long", at == len(long_toks))) if done]
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        if "short" in ended:
            fed_short = len(short_toks) + 1
    return steps


@pytest.fixture(scope="module")
def setup(tmp_path_factory):
    long_toks = H.random_tokens(CFG["vocab_size"], N_LONG + N_DECODE, 1)
    short_toks = H.random_tokens(CFG["vocab_size"], 70 + 12, 2)
    return {"long": long_toks, "short": short_toks, "tmp": tmp_path_factory.mktemp("long")}


def run_engine(folder, dtype, setup):
    from spite_amd.engine.engine import Engine
    chunk_pages = -(-(CHUNK + PORTION) // PAGE) + 1            # what the chunked layers may hold, plus the short request
    full_pages = -(-(N_LONG + N_DECODE) // PAGE)
    extra = -(-len(setup["short"]) // PAGE)
    eng = Engine(folder, dtype=dtype, page_size=PAGE, num_pages=[chunk_pages + extra, full_pages + extra],
                 max_requests=2, max_batch_tokens=PORTION + 1)
    assert eng.cache.groups[0].key[2] == "chunk" and eng.cache.groups[1].key[2] == "full"
    steps = schedule(setup["long"], setup["short"])
    assert any(len(s["entries"]) == 2 and len(s["entries"][1]["tokens"]) == PORTION for s in steps)
    routing, peak = {}, 0
    from spite_amd.engine.engine import StepEntry
    slots, out = {}, {}
    for rec in steps:
        entries = []
        for e in rec["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = eng.admit()
            entries.append(StepEntry(slots[e["id"]], e["tokens"], e["want"]))
        for e in entries:                           # what the step will hold while it runs
            eng.cache.reserve(e.slot, len(e.tokens))
        if "long" in slots:
            peak = max(peak, sum(p >= 0 for p in eng.cache.block_table(slots["long"], 0)))
        trace = {}
        logits = eng.step(entries, trace=trace)
        out[rec["step"]] = logits.cpu().numpy().copy()
        routing[rec["step"]] = [t.cpu().numpy() for t in trace.get("moe_experts", [])]
        for rid in rec["end"]:
            eng.release(slots.pop(rid))
        eng.cache.check()
    # the chunked group never held more than a chunk and a portion of the long request
    assert peak <= chunk_pages, (peak, chunk_pages)
    assert peak >= CHUNK // PAGE
    for g in range(eng.cache.n_groups()):
        assert eng.cache.free_pages(g) == eng.cache.total_pages(g)
    return H.collect(steps, out, CFG["vocab_size"]), H.routing_hints(CFG, steps, routing)


def reference(weights, setup, hints=None, hint_rel=0.0, taken=None, cfg=CFG):
    rows = {}
    want_long = wanted_positions() + list(range(N_LONG, N_LONG + N_DECODE))
    n_prompt_short = len(setup["short"]) - 12
    want_short = list(range(n_prompt_short - 1, len(setup["short"])))
    for rid, toks, want in (("long", setup["long"], want_long), ("short", setup["short"], want_short)):
        took = []
        out = plain.forward(cfg, weights, toks, rows=want, route_hints=None if hints is None else hints[rid],
                            hint_rel=hint_rel, taken=took, rope_angle_dtype=torch.float32).to(torch.float32).numpy()
        if taken is not None:
            taken.extend((rid, L, t) for L, t in took)
        for i, p in enumerate(want):
            rows[(rid, p)] = out[i]
    return rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_seventeen_thousand_tokens_in_portions_then_decoded(dtype, setup):
    folder = str(setup["tmp"] / dtype)
    from spite_amd.weights.random_init import write_random_model
    write_random_model(folder, CFG, 3, dtype=dtype, overrides=planted(3))
    weights = H.read_weights(folder)
    got, hints = run_engine(folder, dtype, setup)
    taken = []
    if dtype == "float32":
        ref = reference(weights, setup)
    else:
        ref = reference(weights, setup, hints, TOL_BF16_REL, taken)
    scale = max(float(np.abs(v).max()) for v in ref.values())
    tol = TOL_F32 if dtype == "float32" else TOL_BF16_REL * scale
    d, where = H.max_diff(got, ref)
    n_tok = (N_LONG + N_DECODE + len(setup["short"])) * 3
    print(f"\n[long {dtype}] {len(ref)} rows: max|diff| vs plain {d:.3e} at {where} (tol {tol:.3e}, scale {scale:.2f}); "
          f"{len(taken)} of {n_tok} routing choices followed as near ties")
    assert d <= tol, f"{d} at {where}"
    assert len(taken) <= 0.03 * n_tok
    setup[dtype] = (got, weights)


def test_a_wrong_chunk_or_temperature_is_visible(setup):
    # the check above has teeth: the plain implementation with another chunk size, without the
    # temperature, or with a window instead of chunks differs from the engine's 32-bit logits by far
    # more than the bfloat16 tolerance, at positions beyond the first chunk
    if "float32" not in setup:
        pytest.skip("needs the 32-bit run of the test above")
    got, weights = setup["float32"]
    scale = max(float(np.abs(v).max()) for v in got.values())
    want = [p for p in wanted_positions() if p >= CHUNK][:40]
    mine = np.stack([got[("long", p)] for p in want])
    for label, cfg in (("chunk of 8256", dict(CFG, attention_chunk_size=CHUNK + 64)),
                       ("no temperature", dict(CFG, attn_temperature_tuning=False)),
                       ("floor_scale 4096", dict(CFG, floor_scale=4096)),
                       ("window", dict(CFG, attention_local_kind="window"))):
        other = plain.forward(cfg, weights, setup["long"][:want[-1] + 1], rows=want,
                              rope_angle_dtype=torch.float32).to(torch.float32).numpy()
        d = float(np.abs(other - mine).max())
        print(f"\n[long] plain with {label}: differs by {d:.3e} ({d / scale:.1%} of the scale)")
        # the temperature's other step is a change of 4 % in the queries' scale: the 32-bit run
        # sees it a thousand times over; the bfloat16 run's tolerance is as large as it
        assert d > (1000 * TOL_F32 if label.startswith("floor_scale") else 2.5 * TOL_BF16_REL * scale), label
