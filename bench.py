#!/usr/bin/env python3
"""Measures generation on one MI355X: decode tokens a second at batch 8 (the headline),
batch 1 and batch 64, and the prefill of a 2,048-token prompt, on the layer sizes of Llama 4
Scout with random weights, and prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L]

A "step" is one decode step of the whole batch through the engine's own step function and
sampler (greedy), the sampled tokens fed back.  The requests' context (4,096 positions each)
is put into the cache before the timed region by filling the pages with random values: the
timed steps read it as they would read a real context.  The prefill is timed on its own.
Roofline: bytes that a decode step has to read (every weight it uses once, the cache of the
live requests) / its time, against 8 TB/s; prefill FLOPs / time against 2.5 PFLOP/s bf16.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12          # bytes/s
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

SCOUT = dict(
    architectures=["Llama4ForCausalLM"], num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
    num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5, num_local_experts=16, num_experts_per_tok=1,
    intermediate_size=8192, intermediate_size_mlp=16384, interleave_moe_layer_step=1, vocab_size=202048,
    tie_word_embeddings=False, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=16.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    attention_chunk_size=8192, use_qk_norm=True, attn_temperature_tuning=True, floor_scale=8192, attn_scale=0.1,
    torch_dtype="bfloat16")
TINY = dict(SCOUT, num_hidden_layers=4, hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
            intermediate_size=512, intermediate_size_mlp=1024, vocab_size=4096, num_local_experts=4)


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def layer_bytes(cfg, item=2):
    d, H, G, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    F, E = cfg["intermediate_size"], cfg["num_local_experts"]
    attn = ((H + 2 * G) * hd * d + d * H * hd) * item
    expert = 3 * d * F * item
    router = E * d * 4
    norms = 2 * d * 4
    return attn, expert, router + norms


def decode_bytes(cfg, L, batch, context, experts_touched, item=2):
    """Bytes one decode step has to read: every weight it uses once and the cache that the live
    requests' queries can see (every fourth layer the whole context, the others the current
    chunk)."""
    d, V = cfg["hidden_size"], cfg["vocab_size"]
    attn, expert, small = layer_bytes(cfg, item)
    kv_token = 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * item
    chunk = cfg["attention_chunk_size"]
    n_full = sum(1 for layer in range(L) if (layer + 1) % 4 == 0)
    seen = n_full * context + (L - n_full) * (context % chunk + 1 if context >= chunk else context)
    step = cfg["interleave_moe_layer_step"]
    n_moe = sum(1 for layer in range(L) if (layer + 1) % step == 0)
    dense = 3 * d * cfg["intermediate_size_mlp"] * item
    return L * (attn + small) + n_moe * expert * (1 + experts_touched) + (L - n_moe) * dense \
        + batch * seen * kv_token + V * d * item + batch * d * item + d * 4


def visible_pairs(T, past, span=None):
    """(query, key) pairs of a portion of T tokens that follows `past` cached ones: every key up
    to the query itself, or only those of the query's own chunk of `span` positions."""
    if span is None:
        return T * past + T * (T + 1) // 2
    return sum(p % span + 1 for p in range(past, past + T))


def prefill_flops(cfg, L, T, past=0):
    d, H, G, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    F, V = cfg["intermediate_size"], cfg["vocab_size"]
    step = cfg["interleave_moe_layer_step"]
    n_moe = sum(1 for layer in range(L) if (layer + 1) % step == 0)
    proj = (H + 2 * G) * hd * d + d * H * hd
    moe = 2 * 3 * d * F + cfg["num_local_experts"] * d            # one routed expert and the shared one a token
    dense = 3 * d * cfg["intermediate_size_mlp"]
    n_full = sum(1 for layer in range(L) if (layer + 1) % 4 == 0)
    pairs = n_full * visible_pairs(T, past) + (L - n_full) * visible_pairs(T, past, cfg["attention_chunk_size"])
    return L * 2 * proj * T + 4 * pairs * H * hd + 2 * T * (n_moe * moe + (L - n_moe) * dense) + 2 * d * V


def sampling_only(V, rows, steps):
    """Times the sampler alone (no model): rows of random logits, peaked like a trained model's or
    flat like a random one's, through the option sets that the command line offers."""
    import numpy as np
    import torch
    from spite_amd.sampling.sampler import Sampler, SamplingParams
    dev = torch.device("cuda:0")
    sampler = Sampler(dev)
    g = torch.Generator(device=dev).manual_seed(0)
    out = {}
    for spread, scale in (("peaked", 3.0), ("flat", 0.05)):
        logits = torch.randn(rows, V, device=dev, generator=g) * scale
        for name, p in (("greedy", SamplingParams()), ("temperature", SamplingParams(temperature=0.8)),
                        ("top_p", SamplingParams(temperature=0.8, top_p=0.95)),
                        ("top_k", SamplingParams(temperature=0.8, top_k=40)),
                        ("all", SamplingParams(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repetition_penalty=1.1))):
            params, ctx, st = [p] * rows, [[1, 2, 3]] * rows, [1] * rows
            for _ in range(2):
                sampler.sample(logits, params, ctx, st)
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(steps):
                sampler.sample(logits, params, ctx, st)
            torch.cuda.synchronize()
            out[f"{spread}_{name}_ms"] = round((time.perf_counter() - t) / steps * 1e3, 3)
            log(f"sampling {rows} rows of {V}, {spread} logits, {name}: {out[f'{spread}_{name}_ms']} ms a call")
    print(json.dumps({"metric": "sampling only", "value": None, "n_gpus": 1, "rows": rows, "vocab": V, "ms_per_call": out}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (memory or time)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--prefill-context", type=int, default=0,
                    help="the timed prompt portion follows this many tokens already in the cache")
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--tiny", action="store_true", help="a small model of the same kind, to try the script")
    ap.add_argument("--experts", type=int, default=None, help="routed experts a layer (default: the model's 16)")
    ap.add_argument("--moe-step", type=int, default=None,
                    help="every how many layers the feed-forward is the experts' (default 1; 2 = dense layers between)")
    ap.add_argument("--no-graphs", action="store_true", help="run decode steps eagerly (for kernel traces)")
    ap.add_argument("--phase", default="all", choices=["all", "decode", "prefill", "sampling"],
                    help="time only one phase (for kernel traces); the other's figures are null")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import numpy as np
    import torch
    from spite_amd.engine.engine import Engine, StepEntry
    from spite_amd.sampling.sampler import Sampler, SamplingParams

    base = TINY if args.tiny else SCOUT
    if args.phase == "sampling":
        return sampling_only(base["vocab_size"], args.batch, args.steps)
    layers_full = base["num_hidden_layers"]
    L = args.layers or layers_full
    cfg = dict(base, num_hidden_layers=L, no_rope_layers=None)
    if args.experts:
        cfg["num_local_experts"] = args.experts
    if args.moe_step:
        cfg["interleave_moe_layer_step"] = args.moe_step
    item = 2 if args.dtype == "bf16" else 4
    points = [int(x) for x in args.points.split(",") if x.strip()]
    max_b = max([args.batch] + points)
    page = 64
    per_req = -(-(args.context + args.steps + args.warmup + 8) // page) * page
    cache_tokens = max(max_b * per_req, args.prefill_context + args.prefill_tokens + 2 * page)
    log(f"building {L} of {layers_full} layers, cache for {cache_tokens} positions")
    t0 = time.time()
    eng = Engine(cfg, dtype=args.dtype, page_size=page, cache_tokens=cache_tokens, max_requests=max_b,
                 max_batch_tokens=max(args.prefill_tokens, max_b), random_weights=True, seed=0,
                 graphs=not args.no_graphs)
    torch.cuda.synchronize()
    log(f"model and cache on the GPU in {time.time() - t0:.1f} s, "
        f"{torch.cuda.memory_allocated() / 2**30:.1f} GiB allocated")
    V = cfg["vocab_size"]
    rng = np.random.RandomState(0)
    sampler = Sampler(eng.device)

    # ---- prefill of one prompt
    def prefill_once():
        s = eng.admit()
        if args.prefill_context:
            eng.cache.reserve(s, args.prefill_context)
            eng.cache.commit(s, args.prefill_context)
        toks = rng.randint(0, V, size=args.prefill_tokens).tolist()
        torch.cuda.synchronize()
        t = time.perf_counter()
        logits = eng.step([StepEntry(s, toks, [len(toks) - 1])])
        sampler.sample(logits, [SamplingParams()], [toks], [0])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        eng.release(s)
        return dt
    prefill = None
    if args.phase != "decode":
        if args.prefill_context:
            for g in eng.cache.groups:
                g.kv.normal_(0.0, 1.0)
        prefill_once()
        pre = min(prefill_once() for _ in range(2))
        pf = prefill_flops(cfg, L, args.prefill_tokens, args.prefill_context)
        prefill = {"value": round(args.prefill_tokens / pre, 1), "tokens": args.prefill_tokens,
                   "ms": round(pre * 1e3, 3), "frac": round(pf / pre / MFMA_PEAK[args.dtype], 4)}
        if args.prefill_context:
            prefill["after"] = args.prefill_context
        log(f"prefill {args.prefill_tokens} tokens" + (f" after {args.prefill_context}" if args.prefill_context else "")
            + f": {pre * 1e3:.1f} ms")
    if args.phase == "prefill":
        print(json.dumps({"metric": "prefill only", "value": None, "prefill": prefill, "n_gpus": 1,
                          "config": {"layers": L, "layers_full": layers_full}}))
        return 0

    # ---- decode at a fixed batch
    def fill_context(slots):
        for s in slots:
            eng.cache.reserve(s, args.context)
            eng.cache.commit(s, args.context)
        for g in eng.cache.groups:
            g.kv.normal_(0.0, 1.0)

    def decode(batch, steps, warmup):
        slots = [eng.admit() for _ in range(batch)]
        fill_context(slots)
        toks = rng.randint(0, V, size=batch).tolist()
        params = [SamplingParams() for _ in range(batch)]
        ctxs = [[] for _ in range(batch)]
        states = [0] * batch
        experts = []

        def one(trace=None):
            nonlocal toks
            logits = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)], trace=trace)
            toks = sampler.sample(logits, params, ctxs, states)
        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        trace = {}
        one(trace)
        for e in trace.get("moe_experts", []):
            experts.append(len(set(e.cpu().tolist())))
        for s in slots:
            eng.release(s)
        return dt, (sum(experts) / len(experts) if experts else 0.0)

    dt, touched = decode(args.batch, args.steps, args.warmup)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    nbytes = decode_bytes(cfg, L, args.batch, args.context + args.warmup + args.steps // 2, touched, item)
    achieved = nbytes / (dt / args.steps)
    log(f"decode batch {args.batch}: {ms:.2f} ms/step, {value:.1f} tok/s, {touched:.1f} experts a layer")
    pts = {}
    for b in points:
        n = max(4, args.steps // 2)
        d_b, _ = decode(b, n, 2)
        pts[f"decode_b{b}"] = round(b * n / d_b, 1)
        log(f"decode batch {b}: {d_b / n * 1e3:.2f} ms/step")

    out = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} "
                  f"({'a tiny Llama 4 shape' if args.tiny else 'Llama 4 Scout shape'}, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0,0.02), uniform-random token ids, "
                                     "context pages filled with random values",
        "config": {"model": "llama4-scout-shape" if not args.tiny else "llama4-tiny-shape", "layers": L,
                   "layers_full": layers_full, "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "experts": cfg["num_local_experts"], "moe_every": cfg["interleave_moe_layer_step"], "top_k": 1,
                   "expert_intermediate": cfg["intermediate_size"],
                   "shared_expert": 1, "vocab": V, "chunk": cfg["attention_chunk_size"], "nope_every": 4,
                   "global_batch": args.batch, "seq_len": args.context, "page_size": page,
                   "parallelism": "none (1 GPU)"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": pts,
        "peak_memory_gib": round(torch.cuda.max_memory_allocated() / 2**30, 1),
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
