"""generate(): requests in, tokens out, through the scheduler, the step function and the
sampler.  The loop of crates/spite-executor/src/lib.rs:640-678 (prefill, then sample and
decode until ``max_tokens`` or an end-of-sequence token, which is not emitted), for many
requests at once."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

from ..sampling.sampler import Sampler, SamplingParams
from .engine import StepEntry
from .scheduler import Scheduler


@dataclass
class GenerationResult:
    tokens: List[int] = field(default_factory=list)
    finish_reason: str = "NotDone"
    n_prompt: int = 0


def generate(engine, prompts: Sequence[Sequence[int]], max_tokens: int = 16, temperature: float = 0.0,
             seed: int = 0, top_k: int = 0, top_p: float = 1.0, min_p: float = 0.0,
             repetition_penalty: float = 1.0, repeat_last_n: int = 64, stop_token_ids: Sequence[int] = (),
             eos_token_ids: Optional[Sequence[int]] = None, max_context: Optional[int] = None,
             max_batch_tokens: Optional[int] = None, details: bool = False, stats: Optional[dict] = None,
             timeline: Optional[list] = None):
    """Generated token ids of every prompt (lists of ints).  Request i draws from its own
    random stream seeded ``seed ^ i``, so its tokens do not depend on the other requests.
    With ``details`` the results carry the finish reason.  ``stats`` (a dict) receives the
    counts of steps, tokens and preemptions, the time to every request's first token
    (``ttft_s``, in the order of the prompts, from the call's start) and the most pages that
    each group of layers held (``peak_pages``).  ``timeline`` (a list) receives one record a
    step: wall seconds, GPU seconds between the step's first and last kernel, prompt tokens and
    decoded tokens in it and the position at which every entry began (the sampled tokens come
    back to the host every step, so a step's wall time includes all of its GPU work)."""
    import time
    import torch
    t_begin = time.perf_counter()
    eos = list(engine.spec.eos_token_ids) if eos_token_ids is None else list(eos_token_ids)
    ctx_limit = int(max_context) if max_context is not None else engine.spec.max_position
    sched = Scheduler(engine.cache, max_batch_tokens or engine.max_batch_tokens, ctx_limit, eos)
    sampler = Sampler(engine.device)
    results: Dict[int, GenerationResult] = {}
    order: List[int] = []
    params: Dict[int, SamplingParams] = {}
    rng: Dict[int, int] = {}
    context: Dict[int, List[int]] = {}
    for i, prompt in enumerate(prompts):
        rid = sched.submit(list(prompt), max_tokens, stop_token_ids)
        order.append(rid)
        results[rid] = GenerationResult(n_prompt=len(prompt))
        params[rid] = SamplingParams(temperature, top_k, top_p, min_p, repetition_penalty, repeat_last_n, seed)
        rng[rid] = (int(seed) ^ i) & ((1 << 64) - 1)
        context[rid] = list(prompt)
    n_steps = n_tokens = 0
    first_token: Dict[int, float] = {}
    cache = engine.cache
    peak = [0] * cache.n_groups()
    while sched.active_count() > 0:
        t_step = time.perf_counter()
        batch = sched.schedule()
        if not batch:
            outs = sched.update([])
            if not outs:
                raise RuntimeError("scheduler made no progress")
        else:
            entries = [StepEntry(b.slot, b.tokens, [len(b.tokens) - 1] if b.wants_logits else []) for b in batch]
            for g in range(len(peak)):           # the scheduler has reserved this step's pages
                peak[g] = max(peak[g], cache.total_pages(g) - cache.free_pages(g))
            if timeline is not None:
                ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                ev0.record()
            logits = engine.step(entries, commit=False)
            wanted = [b.request_id for b in batch if b.wants_logits]
            states = [rng[r] for r in wanted]
            toks = sampler.sample(logits, [params[r] for r in wanted], [context[r] for r in wanted], states, keys=wanted)
            for r, s in zip(wanted, states):
                rng[r] = s
            if timeline is not None:
                ev1.record()
                ev1.synchronize()      # a step that wants no logits would else end before its kernels have run
            outs = sched.update(toks)
            n_steps += 1
            n_tokens += sum(len(b.tokens) for b in batch)
            now = time.perf_counter()
            for r in wanted:
                first_token.setdefault(r, now - t_begin)
            if timeline is not None:
                timeline.append({"wall_s": now - t_step, "gpu_s": ev0.elapsed_time(ev1) * 1e-3,
                                 "prompt_tokens": sum(len(b.tokens) for b in batch if b.start < results[b.request_id].n_prompt),
                                 "decoded_tokens": sum(1 for b in batch if b.start >= results[b.request_id].n_prompt),
                                 "entries": len(batch), "starts": [b.start for b in batch]})
        for o in outs:
            res = results[o.request_id]
            if o.token >= 0:
                res.tokens.append(o.token)
                context[o.request_id].append(o.token)
            if o.done:
                res.finish_reason = o.finish_reason
                sampler.forget(o.request_id)
    if stats is not None:
        stats.update(steps=n_steps, tokens=n_tokens, preemptions=sched.n_preemptions,
                     ttft_s=[first_token.get(r) for r in order], peak_pages=peak,
                     seconds=time.perf_counter() - t_begin)
    if details:
        return [results[r] for r in order]
    return [results[r].tokens for r in order]
