#!/usr/bin/env python3
"""Measures generation on one MI355X and prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--runs R] [--workload decode|longctx|serve]

``decode`` (the default, the headline): decode tokens a second at batch 8, batch 1 and batch
64, and the prefill of a 2,048-token prompt, on the layer sizes of Llama 4 Scout with random
weights.  A "step" is one decode step of the whole batch through the engine's own step function
and sampler (greedy), the sampled tokens fed back.  The requests' context (4,096 positions
each) is put into the cache before the timed region by filling the pages with random values: the
timed steps read it as they would read a real context.  K steps are timed R times; ``value``
and ``ms_per_step`` are the median run's, ``runs_ms`` lists all.
Roofline: bytes that a decode step has to read (every weight it uses once, the cache of the
live requests) / its time against 8 TB/s, and against what a plain streaming read reaches on
this GPU, measured before the run; prefill FLOPs / time against 2.5 PFLOP/s bf16, and against
what this library's own large dense product reaches.

``longctx``: 16 layers of Scout's sizes, 8 requests of 30,000 random tokens fed by the
scheduler in portions of 2,048 (pages roll off behind the chunk of 8,192 on the rotating
layers), then 64 decoded tokens each, through ``Engine.generate``.
``serve``: 12 layers with 128 experts in every second layer, 32 requests with prompts of 512
to 2,048 tokens, 64 new tokens each: decoded tokens lead prompt portions in mixed steps.
Both run three times (``--runs``) and report the median repetition: prefill and decode tokens
a second, the decode steps against the bytes they have to read, time to first token,
step-time percentiles and the most pages held per group of layers; ``longctx`` then decodes 64
tokens with all of its requests live at the prompt's length.  The default run carries both,
shortened, under ``workloads`` (``--no-workloads`` leaves them out).
"""
import argparse
import json
import os
import statistics
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


class Sizes:
    """Bytes and FLOPs of a step, from the typed configuration (which layers rotate, which have
    experts, the chunk: nothing is assumed here)."""

    def __init__(self, typed, item):
        c = self.c = typed
        self.item = item
        d, H, G, hd = c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim
        self.L = c.num_hidden_layers
        self.proj = (H + 2 * G) * hd * d + d * H * hd                 # elements of a layer's attention matrices
        self.expert = 3 * d * c.intermediate_size                      # of one expert
        self.dense = 3 * d * c.intermediate_size_mlp
        self.small = (c.num_local_experts * d + 2 * d) * 4             # router and norms, 32-bit
        self.kv_token = 2 * G * hd * item
        self.n_moe = len(set(c.moe_layers))
        self.full_layers = [i for i in range(self.L) if not c.no_rope_layers[i] or not c.attention_chunk_size]
        self.local_layers = [i for i in range(self.L) if i not in self.full_layers]
        self.span, self.local_kind = c.attention_chunk_size, c.attention_local_kind

    def seen(self, context):
        """Keys that one query at position ``context`` reads, summed over the layers."""
        if not self.local_layers:
            return self.L * context
        local = (context % self.span + 1) if self.local_kind == "chunk" else min(context + 1, self.span)
        return len(self.full_layers) * context + len(self.local_layers) * min(local, context + 1)

    def decode_bytes(self, batch, context, experts_touched):
        c, it = self.c, self.item
        moe_bytes = self.n_moe * (self.expert * it * (1 + experts_touched) + c.num_local_experts * c.hidden_size * 4)
        return (self.L * (self.proj * it + 2 * c.hidden_size * 4) + moe_bytes + (self.L - self.n_moe) * self.dense * it
                + batch * self.seen(context) * self.kv_token + c.vocab_size * c.hidden_size * it
                + batch * c.hidden_size * it + c.hidden_size * 4)

    def decode_bytes_at(self, contexts, experts_touched):
        """As ``decode_bytes`` for requests at positions of their own."""
        b = len(contexts)
        return self.decode_bytes(b, 0, experts_touched) - b * self.seen(0) * self.kv_token \
            + sum(self.seen(c) for c in contexts) * self.kv_token

    def pairs(self, T, past):
        full = T * past + T * (T + 1) // 2
        if not self.local_layers:
            return self.L * full
        if self.local_kind == "chunk":
            local = sum(p % self.span + 1 for p in range(past, past + T))
        else:
            local = sum(min(p + 1, self.span) for p in range(past, past + T))
        return len(self.full_layers) * full + len(self.local_layers) * local

    def prefill_flops(self, T, past=0, logit_rows=1):
        c = self.c
        moe = 2 * self.expert + c.num_local_experts * c.hidden_size   # one routed expert and the shared one a token
        return (self.L * 2 * self.proj * T + 4 * self.pairs(T, past) * c.num_attention_heads * c.head_dim
                + 2 * T * (self.n_moe * moe + (self.L - self.n_moe) * self.dense)
                + 2 * c.hidden_size * c.vocab_size * logit_rows)


def measured_peaks(dtype):
    """What this GPU gives to the simplest kernels of the same kind: a streaming read of 4 GiB
    (non-temporal loads, a contiguous piece per workgroup), this library's dense product at
    8192^3, and a loop of MFMAs alone on random and on zero operands; the best of a few runs each."""
    import torch
    from spite_amd.csrc import hipops
    dev = torch.device("cuda:0")
    buf = torch.empty(1 << 30, dtype=torch.float32, device=dev).normal_()
    best = 0.0
    for blocks in (512, 1024, 4096):
        out = torch.zeros(8 * blocks, dtype=torch.float32, device=dev)
        for _ in range(4):
            torch.cuda.synchronize()
            t = time.perf_counter()
            hipops.stream_read(buf, out)
            torch.cuda.synchronize()
            best = max(best, buf.numel() * 4 / (time.perf_counter() - t))
    del buf
    res = {"hbm_read_GBps": round(best / 1e9, 1)}
    if dtype == "bf16":
        n = 8192
        a = torch.randn(n, n, device=dev).to(torch.bfloat16)
        w = hipops.operand_order(torch.randn(n, n, device=dev).to(torch.bfloat16))
        y = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
        rate = 0.0
        for _ in range(6):
            torch.cuda.synchronize()
            t = time.perf_counter()
            hipops.gemm_tiled(a, w, y, n, n, n)
            torch.cuda.synchronize()
            rate = max(rate, 2.0 * n ** 3 / (time.perf_counter() - t))
        res["dense_product_TFLOPs"] = round(rate / 1e12, 1)
        # the matrix units alone, operands in registers: on pseudo-random values and on zeros (the
        # difference is the chip's power limit, which real values meet and zeros do not)
        out = torch.zeros(1024, dtype=torch.float32, device=dev)
        for label, gain in (("mfma_loop_random_TFLOPs", 1.0), ("mfma_loop_zeros_TFLOPs", 0.0)):
            rate = 0.0
            for _ in range(3):
                torch.cuda.synchronize()
                t = time.perf_counter()
                flops = hipops.mfma_loop(out, 4000, gain)
                torch.cuda.synchronize()
                rate = max(rate, flops / (time.perf_counter() - t))
            res[label] = round(rate / 1e12, 1)
    torch.cuda.empty_cache()
    return res


class KernelTimes:
    """Wraps every launching function of the kernel binding with a pair of events: the time share
    of each kind of kernel in eager steps, without a profiler."""

    NAMES = ("embed", "add_rmsnorm", "rope_kvwrite", "router_top1", "moe_plan", "convert", "gemm_generic",
             "attn_generic", "gemm_skinny", "gemm_mfma", "gemm_tiled", "attn_decode", "attn_prefill",
             "sample_rows", "argmax_rows", "filter_rows")

    def __init__(self):
        import torch
        from spite_amd.csrc import hipops
        self.torch, self.hipops, self.saved, self.events = torch, hipops, {}, []

    def __enter__(self):
        for name in self.NAMES:
            fn = getattr(self.hipops, name)
            self.saved[name] = fn

            def wrapped(*a, fn_=fn, name_=name, **kw):
                e0, e1 = self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)
                label = name_
                if name_.startswith("gemm"):
                    label = f"{name_} N={a[4]} K={a[5]}" + (" glu" if kw.get("glu") else "") + \
                        (" grouped" if kw.get("offsets") is not None else "")
                e0.record()
                r = fn_(*a, **kw)
                e1.record()
                self.events.append((label, e0, e1))
                return r
            setattr(self.hipops, name, wrapped)
        return self

    def __exit__(self, *exc):
        for name, fn in self.saved.items():
            setattr(self.hipops, name, fn)

    def table(self, steps):
        self.torch.cuda.synchronize()
        tot = {}
        for label, e0, e1 in self.events:
            t, n = tot.get(label, (0.0, 0))
            tot[label] = (t + e0.elapsed_time(e1), n + 1)
        whole = sum(t for t, _ in tot.values()) or 1.0
        rows = sorted(tot.items(), key=lambda kv: -kv[1][0])
        return [{"kernel": k, "ms_per_step": round(t / steps, 4), "calls_per_step": round(n / steps, 1),
                 "share": round(t / whole, 4)} for k, (t, n) in rows]


def sampling_only(V, rows, steps):
    """Times the sampler alone (no model): rows of random logits, peaked like a trained model's or
    flat like a random one's, through the option sets that the command line offers."""
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


def percentiles(xs):
    xs = sorted(xs)
    if not xs:
        return None
    at = lambda q: xs[min(len(xs) - 1, int(q * len(xs)))]
    return {"n": len(xs), "p50": round(at(0.5) * 1e3, 3), "p90": round(at(0.9) * 1e3, 3), "max": round(xs[-1] * 1e3, 3)}


def config_record(cfg, typed, L, layers_full, **more):
    """The sizes of the run, flat."""
    rec = {"model": more.pop("model"), "layers": L, "layers_full": layers_full, "hidden": cfg["hidden_size"],
           "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
           "experts": cfg["num_local_experts"], "moe_every": cfg["interleave_moe_layer_step"], "top_k": 1,
           "expert_intermediate": cfg["intermediate_size"], "dense_intermediate": cfg["intermediate_size_mlp"],
           "shared_expert": 1, "vocab": cfg["vocab_size"], "chunk": typed.attention_chunk_size,
           "nope_layers": sum(1 for x in typed.no_rope_layers if not x)}
    rec.update(more)
    rec["parallelism"] = "none (1 GPU)"
    return rec


def expected_experts(batch, E):
    """How many of E experts b tokens touch when every token picks one uniformly."""
    return E * (1.0 - (1.0 - 1.0 / E) ** batch)


def timed_decode(eng, sampler, typed, batch, context, steps, warmup, n_runs, V, rng, kernel_times=False):
    """Decode steps of ``batch`` requests whose cache holds ``context`` positions each (pages
    taken as a prompt's portions would take them and filled with random values), the sampled
    tokens fed back: seconds of each of ``n_runs`` runs of ``steps`` steps, the experts touched
    a layer (traced steps after the timed ones), and per-kernel shares if asked for."""
    import torch
    from spite_amd.engine.engine import StepEntry
    from spite_amd.sampling.sampler import SamplingParams
    slots = [eng.admit() for _ in range(batch)]
    for s in slots:                       # in portions, as a prompt would come: pages roll off behind the chunk
        for at in range(0, context, 2048):
            n = min(2048, context - at)
            eng.cache.reserve(s, n)
            eng.cache.commit(s, n)
    for g in eng.cache.groups:
        for half in g.halves():
            half.normal_(0.0, 1.0)
    toks = rng.randint(0, V, size=batch).tolist()
    params = [SamplingParams() for _ in range(batch)]
    ctxs = [[] for _ in range(batch)]
    states = [0] * batch

    def one(trace=None):
        nonlocal toks
        logits = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)], trace=trace)
        toks = sampler.sample(logits, params, ctxs, states)
    for _ in range(warmup):
        one()
    times = []
    for _ in range(n_runs):
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
    # how many experts a layer's tokens touch: traced steps (eager, the routers' choices read
    # back once at the end) that go on from the timed ones
    traces = []
    for _ in range(min(steps, 16)):
        traces.append({})
        one(traces[-1])
    counts = [torch.stack([torch.bincount(e.long(), minlength=typed.num_local_experts).gt(0).sum()
                           for e in tr.get("moe_experts", [])]) for tr in traces if tr.get("moe_experts")]
    touched = float(torch.stack(counts).float().mean()) if counts else 0.0
    table = None
    if kernel_times:
        graphs, eng.use_graphs = eng.use_graphs, False
        with KernelTimes() as kt:
            for _ in range(4):
                one()
            table = kt.table(4)
        eng.use_graphs = graphs
    for s in slots:
        eng.release(s)
    return times, touched, table


def serving_workload(args, base, Engine, reps=3):
    """``longctx`` and ``serve``: whole requests through the scheduler, the step function and the
    sampler (``Engine.generate``): one untimed warm-up generation of a few short requests first
    (crates/spite-bench/src/main.rs:257), then the workload ``reps`` times, every step timed
    (:285-305: the prompt steps, then the decode steps); the figures are the median repetition's
    (:331-332).  The steps that only decode are held against the bytes they have to read
    (``Sizes.decode_bytes_at`` of each step's requests and positions).  ``longctx`` ends with a
    phase of its own: all requests live at the prompt's length, 64 tokens decoded together."""
    import numpy as np
    import torch
    from spite_amd.config import read_config
    from spite_amd.sampling.sampler import Sampler
    rng = np.random.RandomState(1)
    layers_full = base["num_hidden_layers"]
    if args.workload == "longctx":
        L = args.layers or 16
        cfg = dict(base, num_hidden_layers=L, no_rope_layers=None)
        n_req, new = args.requests or 8, args.new_tokens or 64
        lens = [args.prompt_tokens or 30000] * n_req
        model = "llama4-scout-shape"
    else:
        L = args.layers or 12
        cfg = dict(base, num_hidden_layers=L, no_rope_layers=None, num_local_experts=args.experts or 128,
                   interleave_moe_layer_step=args.moe_step or 2)
        n_req, new = args.requests or 32, args.new_tokens or 64
        lo, hi = (512, 2048) if not args.prompt_tokens else (args.prompt_tokens // 4, args.prompt_tokens)
        lens = [int(x) for x in rng.randint(lo, hi + 1, size=n_req)]
        model = "llama4-maverick-layer-shapes"
    if args.tiny:
        lens = [max(8, n // 16) for n in lens]
    _, typed = read_config(cfg)
    sizes = Sizes(typed, 2 if args.dtype == "bf16" else 4)
    page, budget = 64, args.prefill_tokens
    # longctx: room for the phase in which all requests decode together (warm-up, the timed runs, traced steps)
    tail = new + 1 if args.workload != "longctx" else 2 + max(1, reps) * new + min(new, 16) + 1
    per_req = -(-(max(lens) + tail) // page) * page
    log(f"{args.workload}: building {L} layers, {n_req} requests of {min(lens)} to {max(lens)} prompt tokens")
    t0 = time.time()
    eng = Engine(cfg, dtype=args.dtype, page_size=page, cache_tokens=n_req * per_req, max_requests=n_req,
                 max_batch_tokens=budget, random_weights=True, seed=0, graphs=not args.no_graphs)
    torch.cuda.synchronize()
    log(f"model and cache on the GPU in {time.time() - t0:.1f} s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB allocated; "
        f"pages per group {[eng.cache.total_pages(g) for g in range(eng.cache.n_groups())]}")
    V = cfg["vocab_size"]
    warm = [rng.randint(0, V, size=min(budget + 3, 300)).tolist() for _ in range(min(n_req, 4))]
    eng.generate(warm, max_tokens=4, eos_token_ids=[])
    prompts = [rng.randint(0, V, size=n).tolist() for n in lens]
    repetitions = []
    for _ in range(max(1, reps)):
        stats, timeline = {}, []
        torch.cuda.synchronize()
        t = time.perf_counter()
        outs = eng.generate(prompts, max_tokens=new, eos_token_ids=[], stats=stats, timeline=timeline)
        torch.cuda.synchronize()
        repetitions.append((time.perf_counter() - t, stats, timeline))
        assert all(len(o) == new for o in outs)
        log(f"{args.workload}: repetition {len(repetitions)}: {repetitions[-1][0]:.2f} s")
    seconds = [r[0] for r in repetitions]
    total, stats, timeline = sorted(repetitions, key=lambda r: r[0])[len(repetitions) // 2]
    kinds = {"prefill": [], "decode": [], "mixed": []}
    for r in timeline:
        kind = "mixed" if r["prompt_tokens"] and r["decoded_tokens"] else "prefill" if r["prompt_tokens"] else "decode"
        kinds[kind].append(r)
    # tokens a second of each kind of work, over the steps that did only that kind
    rate = lambda rs, key: (sum(r[key] for r in rs) / sum(r["wall_s"] for r in rs)) if rs else None
    prefill_tps = rate(kinds["prefill"], "prompt_tokens")
    decode_tps = rate(kinds["decode"], "decoded_tokens")
    host = [r["wall_s"] - r["gpu_s"] for r in timeline]
    n_prompt = sum(lens)
    # the prefill's FLOPs: every request's portions follow its own cached tokens
    flops = 0
    for n in lens:
        for at in range(0, n, budget):
            flops += sizes.prefill_flops(min(budget, n - at), at, logit_rows=0)
    t_prompt = sum(r["wall_s"] for r in kinds["prefill"]) + sum(r["wall_s"] for r in kinds["mixed"])
    # the steps that only decode against the bytes they have to read: every weight they use once
    # (the experts that their tokens are expected to touch) and the cache of their requests
    E = typed.num_local_experts
    dec_bytes = sum(sizes.decode_bytes_at(r["starts"], expected_experts(len(r["starts"]), E)) for r in kinds["decode"])
    dec_time = sum(r["wall_s"] for r in kinds["decode"])
    decode_roof = {"bound": "hbm", "achieved": round(dec_bytes / max(dec_time, 1e-9) / 1e9, 1), "peak": HBM_PEAK / 1e9,
                   "unit": "GB/s", "frac": round(dec_bytes / max(dec_time, 1e-9) / HBM_PEAK, 4),
                   "steps": len(kinds["decode"])} if kinds["decode"] else None
    together = None
    if args.workload == "longctx":
        # every request live at the prompt's length, decoding together
        sampler = Sampler(eng.device)
        ctx_len = max(lens)
        t_d, touched_d, _ = timed_decode(eng, sampler, typed, n_req, ctx_len, new, 2, max(1, reps), V, rng)
        d_med = statistics.median(t_d)
        nb = sizes.decode_bytes(n_req, ctx_len + 2 + new // 2, touched_d)
        together = {"batch": n_req, "context": ctx_len, "steps": new, "tok_s": round(n_req * new / d_med, 1),
                    "ms_per_step": round(d_med / new * 1e3, 3), "frac_of_hbm_peak": round(nb / (d_med / new) / HBM_PEAK, 4),
                    "runs_ms": [round(x / new * 1e3, 3) for x in t_d]}
        log(f"longctx: {n_req} requests decoding together at {ctx_len}: {together['ms_per_step']} ms a step, "
            f"{together['tok_s']} tok/s, {together['frac_of_hbm_peak']} of the HBM peak")
    out = {
        "metric": f"{args.workload}: tokens a second of whole requests through the scheduler "
                  f"({n_req} requests, prompts of {min(lens)} to {max(lens)} tokens, {new} new tokens each)",
        "value": round((n_prompt + n_req * new) / total, 1), "unit": "tok/s", "n_gpus": 1, "steps": len(timeline),
        "warmup": 1, "ms_per_step": round(total / max(len(timeline), 1) * 1e3, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights N(0,0.02), uniform-random token ids",
        "config": config_record(cfg, typed, L, layers_full, model=model, global_batch=n_req, seq_len=max(lens) + new,
                                max_batch_tokens=budget),
        "seconds": round(total, 3), "runs_s": [round(x, 3) for x in seconds],
        "decode_roofline": decode_roof, "decode_together": together,
        "prefill_tps": round(prefill_tps, 1) if prefill_tps else None,
        "decode_tps": round(decode_tps, 1) if decode_tps else None,
        "prompt_frac_of_mfma_peak": round(flops / max(t_prompt, 1e-9) / MFMA_PEAK[args.dtype], 4),
        "ttft_ms": percentiles(stats["ttft_s"]),
        "step_ms": {k: percentiles([r["wall_s"] for r in v]) for k, v in kinds.items()},
        "host_ms_per_step": percentiles(host),
        "peak_pages": stats["peak_pages"],
        "pool_pages": [eng.cache.total_pages(g) for g in range(eng.cache.n_groups())],
        "preemptions": stats["preemptions"],
        "peak_memory_gib": round(torch.cuda.max_memory_allocated() / 2**30, 1),
    }
    log(f"{args.workload}: {total:.2f} s (runs {out['runs_s']}); prefill {out['prefill_tps']} tok/s, decode {out['decode_tps']} tok/s "
        f"({decode_roof['frac'] if decode_roof else None} of the HBM peak), ttft {out['ttft_ms']}, steps {out['step_ms']}, "
        f"host {out['host_ms_per_step']}")
    del eng
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--runs", type=int, default=3, help="how many times the K steps are timed")
    ap.add_argument("--workload", default="decode", choices=["decode", "longctx", "serve"])
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (memory or time)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="tokens of the timed prompt; the scheduler's token budget in the other workloads")
    ap.add_argument("--prefill-context", type=int, default=0,
                    help="the timed prompt portion follows this many tokens already in the cache")
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--tiny", action="store_true", help="a small model of the same kind, to try the script")
    ap.add_argument("--experts", type=int, default=None, help="routed experts a layer (default: the model's 16)")
    ap.add_argument("--moe-step", type=int, default=None,
                    help="every how many layers the feed-forward is the experts' (default 1; 2 = dense layers between)")
    ap.add_argument("--requests", type=int, default=None, help="longctx / serve: how many requests")
    ap.add_argument("--prompt-tokens", type=int, default=None, help="longctx / serve: (longest) prompt")
    ap.add_argument("--new-tokens", type=int, default=None, help="longctx / serve: tokens generated per request")
    ap.add_argument("--no-graphs", action="store_true", help="run decode steps eagerly (for kernel traces)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the measurement of the memory's and the product's rates")
    ap.add_argument("--no-workloads", action="store_true",
                    help="the default run alone, without the longctx and serve workloads behind it")
    ap.add_argument("--kernel-times", action="store_true",
                    help="after the timed runs: eager steps with an event pair around every kernel call, shares per kernel")
    ap.add_argument("--phase", default="all", choices=["all", "decode", "prefill", "sampling"],
                    help="time only one phase (for kernel traces); the other's figures are null")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not measured")
        return 2

    import numpy as np
    import torch
    from spite_amd.config import read_config
    from spite_amd.engine.engine import Engine, StepEntry
    from spite_amd.sampling.sampler import Sampler, SamplingParams

    base = TINY if args.tiny else SCOUT
    if args.phase == "sampling":
        return sampling_only(base["vocab_size"], args.batch, args.steps)
    if args.workload != "decode":
        print(json.dumps(serving_workload(args, base, Engine, args.runs)))
        return 0
    layers_full = base["num_hidden_layers"]
    L = args.layers or layers_full
    cfg = dict(base, num_hidden_layers=L, no_rope_layers=None)
    if args.experts:
        cfg["num_local_experts"] = args.experts
    if args.moe_step:
        cfg["interleave_moe_layer_step"] = args.moe_step
    _, typed = read_config(cfg)
    item = 2 if args.dtype == "bf16" else 4
    sizes = Sizes(typed, item)
    points = [int(x) for x in args.points.split(",") if x.strip()]
    max_b = max([args.batch] + points)
    page = 64
    runs = max(1, args.runs)
    per_req = -(-(args.context + runs * (args.steps + 1) + args.warmup + 8) // page) * page
    cache_tokens = max(max_b * per_req, args.prefill_context + args.prefill_tokens + 2 * page)
    peaks = None
    if not args.no_peaks:
        peaks = measured_peaks(args.dtype)
        log(f"this GPU: streaming read {peaks['hbm_read_GBps']} GB/s"
            + (f", dense product at 8192^3 {peaks['dense_product_TFLOPs']} TFLOP/s" if "dense_product_TFLOPs" in peaks else ""))
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
        for at in range(0, args.prefill_context, 2048):
            n = min(2048, args.prefill_context - at)
            eng.cache.reserve(s, n)
            eng.cache.commit(s, n)
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
                for half in g.halves():
                    half.normal_(0.0, 1.0)
        prefill_once()
        pre_runs = [prefill_once() for _ in range(runs)]
        pre = statistics.median(pre_runs)
        pf = sizes.prefill_flops(args.prefill_tokens, args.prefill_context)
        prefill = {"value": round(args.prefill_tokens / pre, 1), "tokens": args.prefill_tokens,
                   "ms": round(pre * 1e3, 3), "frac": round(pf / pre / MFMA_PEAK[args.dtype], 4),
                   "runs_ms": [round(x * 1e3, 3) for x in pre_runs]}
        if peaks and "dense_product_TFLOPs" in peaks:
            prefill["frac_of_measured_product"] = round(pf / pre / (peaks["dense_product_TFLOPs"] * 1e12), 4)
        if peaks and "mfma_loop_random_TFLOPs" in peaks:
            prefill["frac_of_mfma_on_random_values"] = round(pf / pre / (peaks["mfma_loop_random_TFLOPs"] * 1e12), 4)
        if args.prefill_context:
            prefill["after"] = args.prefill_context
        log(f"prefill {args.prefill_tokens} tokens" + (f" after {args.prefill_context}" if args.prefill_context else "")
            + f": {pre * 1e3:.1f} ms (runs {prefill['runs_ms']})")
        if args.kernel_times:
            with KernelTimes() as kt:
                prefill_once()
                prefill["kernels"] = kt.table(1)
            for row in prefill["kernels"][:12]:
                log(f"  prefill {row['kernel']}: {row['ms_per_step']} ms, {row['share']:.1%}")
    if args.phase == "prefill":
        print(json.dumps({"metric": "prefill only", "value": None, "prefill": prefill, "n_gpus": 1,
                          "config": {"layers": L, "layers_full": layers_full}}))
        return 0

    # ---- decode at a fixed batch
    def decode(batch, steps, warmup, n_runs, kernel_times=False):
        return timed_decode(eng, sampler, typed, batch, args.context, steps, warmup, n_runs, V, rng, kernel_times)

    times, touched, table = decode(args.batch, args.steps, args.warmup, runs, args.kernel_times)
    dt = statistics.median(times)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    mid_context = args.context + args.warmup + (runs * args.steps) // 2
    nbytes = sizes.decode_bytes(args.batch, mid_context, touched)
    achieved = nbytes / (dt / args.steps)
    log(f"decode batch {args.batch}: {ms:.2f} ms/step (runs {[round(x / args.steps * 1e3, 3) for x in times]}), "
        f"{value:.1f} tok/s, {touched:.2f} experts a layer")
    if table:
        for row in table[:12]:
            log(f"  decode {row['kernel']}: {row['ms_per_step']} ms, {row['share']:.1%}")
    pts, pts_roof = {}, {}
    for b in points:
        n = max(4, args.steps // 2)
        t_b, touched_b, _ = decode(b, n, 2, runs)
        d_b = statistics.median(t_b)
        pts[f"decode_b{b}"] = round(b * n / d_b, 1)
        pts_roof[f"decode_b{b}"] = round(sizes.decode_bytes(b, args.context + 2 + (runs * n) // 2, touched_b) / (d_b / n) / HBM_PEAK, 4)
        log(f"decode batch {b}: {d_b / n * 1e3:.2f} ms/step, {touched_b:.2f} experts a layer, {pts_roof[f'decode_b{b}']} of the HBM peak")

    roofline = {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK, 4), "experts_touched": round(touched, 2)}
    if peaks:
        roofline["peak_measured"] = peaks["hbm_read_GBps"]
        roofline["frac_of_measured"] = round(achieved / 1e9 / peaks["hbm_read_GBps"], 4)
    out = {
        "metric": f"decode tok/s at batch {args.batch}, context {args.context} "
                  f"({'a tiny Llama 4 shape' if args.tiny else 'Llama 4 Scout shape'}, random weights)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0,0.02), uniform-random token ids, "
                                     "context pages filled with random values",
        "config": config_record(cfg, typed, L, layers_full, model="llama4-scout-shape" if not args.tiny else "llama4-tiny-shape",
                                global_batch=args.batch, seq_len=args.context, page_size=page),
        "runs": runs, "runs_ms": [round(x / args.steps * 1e3, 3) for x in times],
        "min_ms_per_step": round(min(times) / args.steps * 1e3, 3),
        "prefill": prefill,
        "roofline": roofline,
        "points": pts,
        "points_frac_of_hbm_peak": pts_roof,
        "measured_peaks": peaks,
        "peak_memory_gib": round(torch.cuda.max_memory_allocated() / 2**30, 1),
    }
    if table:
        out["decode_kernels"] = table
    if args.phase == "all" and not args.no_workloads:
        # the other two workloads, on engines of their own once this one's memory is free: whole
        # requests through the scheduler; a failure leaves null and its reason on stderr
        import copy
        import gc
        del eng, sampler
        gc.collect()
        torch.cuda.empty_cache()
        out["workloads"] = {}
        for name in ("longctx", "serve"):
            w_args = copy.copy(args)
            w_args.workload, w_args.layers, w_args.experts, w_args.moe_step = name, None, None, None
            try:
                full = serving_workload(w_args, base, Engine, args.runs)
                keep = ("value", "unit", "seconds", "runs_s", "prefill_tps", "decode_tps", "decode_roofline", "decode_together",
                        "prompt_frac_of_mfma_peak", "ttft_ms", "step_ms", "peak_pages", "pool_pages", "preemptions")
                out["workloads"][name] = dict({k: full[k] for k in keep}, layers=full["config"]["layers"],
                                              experts=full["config"]["experts"], requests=full["config"]["global_batch"],
                                              seq_len=full["config"]["seq_len"])
            except Exception as e:          # noqa: BLE001 - the headline must still be printed
                log(f"workload {name} failed: {type(e).__name__}: {e}")
                out["workloads"][name] = None
            gc.collect()
            torch.cuda.empty_cache()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
