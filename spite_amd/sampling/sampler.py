"""Sampling on the GPU, in the order of the reference's pipeline
(crates/spite-sampling/src/lib.rs:273-296): repetition penalty (window ``repeat_last_n``, each
distinct id once) -> /temperature -> min-p -> top-k -> top-p -> greedy when temperature <= 0,
else the inverse-CDF draw with one LCG stream per request (:343-348).  Names and meanings of
the options are the reference's ``SamplerConfig`` (:83-111); the defaults here switch every
filter off.  Greedy takes the lowest index among equal maxima.  The filters of all rows of a
step run in one kernel (``filter_rows``), the draws in another; the host only packs the options.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..csrc import hipops

LCG_MUL = 6364136223846793005
LCG_ADD = 1442695040888963407
_MASK = (1 << 64) - 1


def lcg_next(state: int):
    """crates/spite-sampling/src/lib.rs:343-348: returns (new state, u in [0,1) as float32)."""
    state = (state * LCG_MUL + LCG_ADD) & _MASK
    return state, float(np.float32(state >> 33) / np.float32(2147483648.0))


@dataclass
class SamplingParams:
    temperature: float = 0.0          # <= 0: greedy
    top_k: int = 0                    # 0 = off
    top_p: float = 1.0                # 1.0 = off
    min_p: float = 0.0                # 0 = off
    repetition_penalty: float = 1.0   # 1.0 = off
    repeat_last_n: int = 64           # 0 = the whole context
    seed: int = 0

    def filters(self) -> bool:
        return (self.top_k > 0 or self.top_p < 1.0 or self.min_p > 0.0
                or abs(self.repetition_penalty - 1.0) >= 1.1920929e-07)


class _Window:
    """The distinct ids among the last ``n`` tokens of one request's context (all of it for
    n = 0), kept up to date token by token instead of being gathered anew every step."""

    def __init__(self, n: int):
        self.n, self.lo, self.hi, self.counts = int(n), 0, 0, {}     # counts: of the tokens at [lo, hi)

    def ids(self, context: Sequence[int], vocab: int) -> List[int]:
        L, n = len(context), self.n
        lo = max(0, L - n) if n else 0
        if L < self.hi or lo >= self.hi:          # another context, or a window that is all new
            self.counts, self.lo, self.hi = {}, lo, lo
        for j in range(self.hi, L):
            t = int(context[j])
            self.counts[t] = self.counts.get(t, 0) + 1
        for j in range(self.lo, lo):              # tokens that left the window
            t = int(context[j])
            c = self.counts[t] - 1
            if c:
                self.counts[t] = c
            else:
                del self.counts[t]
        self.lo, self.hi = lo, L
        return sorted(t for t in self.counts if 0 <= t < vocab)


class Sampler:
    """Keeps what a step needs between steps: the work copy of the logits, one staging buffer on
    either side for the options of all rows (one copy a step), the result's buffers, and, for
    requests that the caller names (``keys``), the penalty window's distinct ids."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._scratch = None
        self._work = None
        self._host = self._dev = None
        self._out = self._out_host = None
        self._windows = {}

    def forget(self, key) -> None:
        """The request ``key`` is over."""
        self._windows.pop(key, None)

    def _staging(self, nbytes: int):
        if self._host is None or self._host.numel() < nbytes:
            size = max(4096, 2 * nbytes)
            self._host = torch.empty(size, dtype=torch.uint8, pin_memory=True)
            self._dev = torch.empty(size, dtype=torch.uint8, device=self.device)
        return self._host, self._dev

    def _penalty_ids(self, p: SamplingParams, context: Sequence[int], key, V: int) -> List[int]:
        if key is None:
            win = context if p.repeat_last_n == 0 or p.repeat_last_n >= len(context) else context[-p.repeat_last_n:]
            return sorted({int(t) for t in win if 0 <= int(t) < V})
        w = self._windows.get(key)
        if w is None or w.n != p.repeat_last_n:
            w = self._windows[key] = _Window(p.repeat_last_n)
        return w.ids(context, V)

    def _pack(self, V: int, params, contexts, rng_states, keys):
        """The options of all rows in one staging buffer and one copy to the GPU:
        [table 6 x n float64 | penalty offsets | penalty ids | temperatures | uniform numbers].
        ``rng_states`` (or None) is advanced for every row that draws."""
        n = len(params)
        filtered = [p.filters() for p in params]
        ids: List[int] = []
        offsets = np.zeros(n + 1, dtype=np.int32)
        table = np.zeros((6, n), dtype=np.float64)
        temps = np.zeros(n, dtype=np.float32)
        us = np.zeros(n, dtype=np.float32)
        for i, p in enumerate(params):
            if filtered[i]:
                table[:, i] = (1.0, max(p.temperature, 0.0), math.log(p.min_p) if p.min_p > 0 else -math.inf,
                               p.top_k if 0 < p.top_k < V else 0, p.top_p, p.repetition_penalty)
                if abs(p.repetition_penalty - 1.0) >= 1.1920929e-07 and len(contexts[i]):
                    ids.extend(self._penalty_ids(p, contexts[i], keys[i] if keys is not None else None, V))
            offsets[i + 1] = len(ids)
            if p.temperature > 0 and rng_states is not None:
                temps[i] = 1.0 if filtered[i] else p.temperature     # filtered rows are divided already
                rng_states[i], us[i] = lcg_next(rng_states[i])
        any_filter, draws = any(filtered), bool(temps.max() > 0)
        if not (any_filter or draws):
            return None, False, False
        parts = [table.reshape(-1).view(np.uint8), offsets.view(np.uint8), np.asarray(ids, dtype=np.int32).view(np.uint8),
                 temps.view(np.uint8), us.view(np.uint8)]
        at, places = 0, []
        for part in parts:
            places.append(at)
            at += (part.size + 15) // 16 * 16
        host, devbuf = self._staging(at)
        hv = host.numpy()
        for place, part in zip(places, parts):
            hv[place:place + part.size] = part
        devbuf[:at].copy_(host[:at], non_blocking=True)
        take = lambda k, dtype, count, item: devbuf[places[k]:places[k] + count * item].view(dtype)
        views = {"table": take(0, torch.float64, 6 * n, 8).view(6, n), "offsets": take(1, torch.int32, n + 1, 4),
                 "ids": take(2, torch.int32, len(ids), 4) if ids else None,
                 "temps": take(3, torch.float32, n, 4), "us": take(4, torch.float32, n, 4)}
        return views, any_filter, draws

    def _filter(self, work: torch.Tensor, params: Sequence[SamplingParams], contexts: Sequence[Sequence[int]], keys=None):
        """Runs the filters of the rows that ask for them over ``work`` in place (one kernel)."""
        views, any_filter, _ = self._pack(work.shape[1], params, contexts, None, keys)
        if any_filter:
            hipops.filter_rows(work, views["table"], views["ids"], views["offsets"])

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], contexts: Sequence[Sequence[int]],
               rng_states: List[int], keys: Optional[Sequence] = None) -> List[int]:
        """One token per row of ``logits`` (fp32 ``[n, V]``).  ``rng_states[i]`` is advanced for
        every row that draws.  ``keys[i]`` names row i's request across steps (its context only
        grows): the penalty window is then kept up to date instead of gathered anew."""
        n, V = logits.shape
        if n == 0:
            return []
        dev = logits.device
        views, any_filter, draws = self._pack(V, params, contexts, rng_states, keys)
        if self._out is None or self._out.numel() < n:
            self._out = torch.empty(max(n, 64), dtype=torch.int32, device=dev)
            self._out_host = torch.empty(max(n, 64), dtype=torch.int32, pin_memory=True)
        out = self._out[:n]
        work = logits
        if any_filter:
            if self._work is None or self._work.shape[0] < n or self._work.shape[1] != V:
                self._work = torch.empty((max(n, 8), V), dtype=torch.float32, device=dev)
            work = self._work[:n]
            work.copy_(logits)
            hipops.filter_rows(work, views["table"], views["ids"], views["offsets"])
        if draws:
            hipops.sample_rows(work, views["temps"], views["us"], out, n)
        else:
            if self._scratch is None or self._scratch[0].numel() < 32 * n:
                self._scratch = (torch.empty(32 * max(n, 64), dtype=torch.float32, device=dev),
                                 torch.empty(32 * max(n, 64), dtype=torch.int32, device=dev))
            hipops.argmax_rows(work, out, self._scratch[0], self._scratch[1], n)
        self._out_host[:n].copy_(out, non_blocking=True)
        torch.cuda.current_stream().synchronize()      # the tokens are wanted on the host now
        return self._out_host[:n].tolist()
