"""Shared by the tests: the two tiny configurations, model folders with planted weights, the
plain implementation's logits, and the replay driver."""
from __future__ import annotations

import json
import os
import subprocess
import sys
import tempfile

import numpy as np
import torch

import plain_llama4 as plain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Two configurations that differ in every size and option.
TINY_A = dict(
    architectures=["Llama4ForCausalLM"], num_hidden_layers=4, hidden_size=64, num_attention_heads=4,
    num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5, num_local_experts=4, num_experts_per_tok=1,
    intermediate_size=128, intermediate_size_mlp=256, interleave_moe_layer_step=1, vocab_size=256,
    rope_theta=500000.0, rope_scaling=None, attention_chunk_size=32, no_rope_layers=[1, 1, 1, 0],
    use_qk_norm=True, attn_temperature_tuning=True, floor_scale=16, attn_scale=0.1,
    tie_word_embeddings=False, torch_dtype="float32")
TINY_B = dict(
    architectures=["Llama4ForCausalLM"], num_hidden_layers=8, hidden_size=96, num_attention_heads=6,
    num_key_value_heads=3, head_dim=24, rms_norm_eps=1e-6, num_local_experts=8, num_experts_per_tok=1,
    intermediate_size=64, intermediate_size_mlp=192, interleave_moe_layer_step=2, vocab_size=384,
    rope_theta=10000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    attention_chunk_size=16, use_qk_norm=False, attn_temperature_tuning=False,
    tie_word_embeddings=False, torch_dtype="float32")
# sizes that the MFMA kernels take (head size 64, pages of 32 keys, widths in operand order):
# the replay tests then run the kernels that serving runs, not their generic stand-ins
TINY_C = dict(
    architectures=["Llama4ForCausalLM"], num_hidden_layers=4, hidden_size=128, num_attention_heads=6,
    num_key_value_heads=2, head_dim=64, rms_norm_eps=1e-5, num_local_experts=4, num_experts_per_tok=1,
    intermediate_size=128, intermediate_size_mlp=192, interleave_moe_layer_step=1, vocab_size=400,
    rope_theta=50000.0, rope_scaling=None, attention_chunk_size=64, no_rope_layers=[1, 0, 1, 1],
    use_qk_norm=True, attn_temperature_tuning=True, floor_scale=32, attn_scale=0.2,
    tie_word_embeddings=False, torch_dtype="float32")
# the reference's own reading of the rotating layers: the last `attention_chunk_size` keys
# (crates/spite-models/src/llama/llama4.rs:189-197) instead of the chunk
TINY_BW = dict(TINY_B, attention_local_kind="window")
TINY_CW = dict(TINY_C, attention_local_kind="window", attention_chunk_size=100)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "Bw": TINY_BW, "Cw": TINY_CW, "Cm": TINY_C}
# "Cm": a bfloat16 folder of C whose shared experts are stored in 32-bit: the engine keeps them so,
# and the shared expert cannot be one more group of the experts' bfloat16 products
KEEP_WIDE = {"Cm": ("shared_expert",)}


def planted_tensors(cfg: dict, seed: int, std: float = 0.05, qk_gain: float = 2.0, router_gain: float = 8.0):
    """Random tensors with the projections of queries and keys and the router scaled up, so
    that attention is far from uniform and the experts are told apart clearly: with plain
    N(0, std) weights a wrong mask or a wrong expert would change the logits very little."""
    from spite_amd.weights.random_init import random_tensors
    # on a GPU box the kernel draws them (the same numbers as the host draws, sooner)
    t = random_tensors(cfg, seed, std, device="cuda:0" if torch.cuda.is_available() else None)
    for name in list(t):
        if name.endswith("q_proj.weight") or name.endswith("k_proj.weight"):
            t[name] = t[name] * qk_gain
        if name.endswith("router.weight"):
            t[name] = t[name] * router_gain
    return t


def make_model(folder: str, cfg: dict, seed: int = 1, dtype: str = "float32", keep_wide=(), **kw) -> dict:
    """Writes a model folder; returns the weights as the file holds them (after rounding to
    the file's dtype), widened to float64, for the plain implementation."""
    from spite_amd.weights.random_init import write_random_model
    write_random_model(folder, cfg, seed, dtype=dtype, overrides=planted_tensors(cfg, seed, **kw), keep_wide=keep_wide)
    return read_weights(folder)


def read_weights(folder: str) -> dict:
    from safetensors.torch import load_file       # a reader that is not the engine's own
    return {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def random_tokens(vocab: int, n: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# ------------------------------------------------------------------ replay
def run_trace_inprocess(engine, steps, routing=None, take=None):
    """Feeds ``steps`` (dicts of the trace format) to an Engine; returns {step: logits[wanted, V]}.
    ``routing`` (a dict) receives {step: [experts of every token, one array per layer with experts]};
    ``take`` (such a dict from another run) makes the engine take those experts."""
    from spite_amd.engine.engine import StepEntry
    slots, out = {}, {}
    for rec in steps:
        entries = []
        for e in rec["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = engine.admit()
            entries.append(StepEntry(slots[e["id"]], e["tokens"], e.get("want", [])))
        trace = {} if routing is not None or take is not None else None
        if take is not None:
            trace["take_experts"] = [torch.from_numpy(np.asarray(t)) for t in take[rec["step"]]]
        logits = engine.step(entries, trace=trace)
        if logits.shape[0]:
            out[rec["step"]] = logits.detach().cpu().numpy().copy()
        if routing is not None:
            routing[rec["step"]] = [t.cpu().numpy() for t in trace.get("moe_experts", [])]
        for rid in rec.get("end", []):
            engine.release(slots.pop(rid))
        engine.cache.check()
    return out


def moe_layers(cfg):
    return [L for L, m in enumerate(plain.layer_kinds(cfg)[1]) if m]


def routing_hints(cfg, steps, routing):
    """{request: {layer: [expert at every position]}} from what a replay recorded."""
    layers = moe_layers(cfg)
    hints = {}
    for rec in steps:
        per_layer = routing[rec["step"]]
        off = 0
        for e in rec["entries"]:
            n = len(e["tokens"])
            h = hints.setdefault(e["id"], {L: [] for L in layers})
            for k, L in enumerate(layers):
                h[L].extend(int(x) for x in per_layer[k][off:off + n])
            off += n
    return hints


def experts_to_take(cfg, steps, hints):
    """{step: [experts of the step's tokens, one array per layer with experts]} from
    {request: {layer: [expert at every position]}}: what ``routing_hints`` returns, cut the way
    ``steps`` cuts the requests."""
    layers = moe_layers(cfg)
    fed, take = {}, {}
    for rec in steps:
        per_layer = [[] for _ in layers]
        for e in rec["entries"]:
            at, n = fed.get(e["id"], 0), len(e["tokens"])
            for k, L in enumerate(layers):
                per_layer[k].extend(hints[e["id"]][L][at:at + n])
            fed[e["id"]] = at + n
        take[rec["step"]] = [np.asarray(x, dtype=np.int32) for x in per_layer]
        for rid in rec.get("end", []):
            fed.pop(rid, None)
    return take


def run_trace_program(model_dir, dtype, steps, max_tokens, extra=(), routing=None):
    """The same through ``bin/trace_run`` as a child process, one step at a time."""
    out_dir = tempfile.mkdtemp(prefix="trace_out_")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *extra]
    if routing is not None:
        cmd.append("--dump-routing")
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {rec['step']}", f"trace_run answered {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    res = {}
    for rec in steps:
        p = os.path.join(out_dir, f"{rec['step']}.f32")
        if os.path.exists(p):
            res[rec["step"]] = np.fromfile(p, dtype="<f4")
        if routing is not None:
            T = sum(len(e["tokens"]) for e in rec["entries"])
            r = np.fromfile(os.path.join(out_dir, f"{rec['step']}.routing.i32"), dtype="<i4")
            routing[rec["step"]] = list(r.reshape(-1, T)) if T else []
    return res


class Collected:
    """Logits gathered from a replay, keyed by (request, position)."""

    def __init__(self, vocab):
        self.vocab, self.rows = vocab, {}

    def add(self, steps, outputs, start_of):
        pos = dict(start_of)
        for rec in steps:
            got = outputs.get(rec["step"])
            k = 0
            for e in rec["entries"]:
                base = pos.get(e["id"], 0)
                for w in e.get("want", []):
                    self.rows[(e["id"], base + w)] = np.asarray(got).reshape(-1, self.vocab)[k]
                    k += 1
                pos[e["id"]] = base + len(e["tokens"])
        return self


def collect(steps, outputs, vocab):
    return Collected(vocab).add(steps, outputs, {}).rows


# ------------------------------------------------------------------ schedules over a set of requests
def schedule_whole(reqs):
    """Each request alone and whole, every position wanted."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(reqs.items())]


def schedule_tail_one_by_one(reqs, tail=32):
    """Most of it in one step, the last ``tail`` tokens one by one."""
    steps, n = [], 0
    for rid, toks in reqs.items():
        head = max(len(toks) - tail, 0)
        if head:
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
            n += 1
        for i in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
            n += 1
    return steps


def schedule_portions(reqs, sizes=(7, 2, 13, 3, 2, 16, 5, 2, 31, 4)):
    """Portions of changing size, down to two tokens, one request at a time."""
    steps, n = [], 0
    for rid, toks in reqs.items():
        at, k = 0, 0
        while at < len(toks):
            sz = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[at:at + sz], "want": list(range(sz))}],
                          "end": [rid] if at + sz == len(toks) else []})
            at += sz
            n += 1
    return steps


def schedule_mixed(reqs, seed=0, max_live=4, portion_sizes=(2, 3, 5, 8, 13), decode_from=0.6):
    """Up to ``max_live`` requests at a time: the first part of each in portions of changing
    size, the rest token by token, portions of some beside single tokens of others; a request
    is sometimes left out of a step.  Requests start as earlier ones end."""
    rng = np.random.RandomState(seed)
    waiting = list(reqs.items())
    live = {}           # id -> [tokens, fed]
    steps, n = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ended = [], []
        ids = list(live)
        rng.shuffle(ids)
        for rid in ids:
            toks, fed = live[rid]
            if len(entries) and rng.rand() < 0.25:
                continue                                   # left out of this step
            if fed >= int(len(toks) * decode_from):
                sz = 1
            else:
                sz = int(portion_sizes[rng.randint(len(portion_sizes))])
            sz = min(sz, len(toks) - fed)
            entries.append({"id": rid, "tokens": toks[fed:fed + sz], "want": list(range(sz))})
            live[rid][1] = fed + sz
            if fed + sz == len(toks):
                ended.append(rid)
        for rid in ended:
            del live[rid]
        steps.append({"step": n, "entries": entries, "end": ended})
        n += 1
    return steps


def plain_logits(cfg, weights, reqs, hints=None, hint_rel=0.0, taken=None, disagreements=None, **kw):
    """{(request, position): logits row} from the plain implementation, whole sequences.
    ``hints``: {request: {layer: experts}} of another implementation (see plain.router_top1)."""
    rows = {}
    for rid, toks in reqs.items():
        took, chosen = [], {}
        out = plain.forward(cfg, weights, toks, route_hints=None if hints is None else hints[rid],
                            hint_rel=hint_rel, taken=took, chosen=chosen, **kw).to(torch.float32).numpy()
        if taken is not None:
            taken.extend((rid, L, t) for L, t in took)
        if disagreements is not None and hints is not None:
            for L, idx in chosen.items():
                disagreements.extend((rid, L, t) for t, (a, b) in enumerate(zip(idx, hints[rid][L])) if a != b)
        for i in range(len(toks)):
            rows[(rid, i)] = out[i]
    return rows


def max_diff(a: dict, b: dict):
    assert a.keys() == b.keys(), f"different rows: {sorted(set(a) ^ set(b))[:5]}"
    worst, where = 0.0, None
    for k in a:
        d = float(np.max(np.abs(a[k].astype(np.float64) - b[k].astype(np.float64))))
        if not np.isfinite(d):
            return float("inf"), k
        if d > worst:
            worst, where = d, k
    return worst, where
