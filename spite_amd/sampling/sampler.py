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
from typing import List, Sequence

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


class Sampler:
    def __init__(self, device):
        self.device = device
        self._scratch = None

    def _filter(self, work: torch.Tensor, params: Sequence[SamplingParams], contexts: Sequence[Sequence[int]]):
        """Runs the filters of the rows that ask for them over ``work`` in place (one kernel)."""
        n, V = work.shape
        table = np.zeros((6, n), dtype=np.float64)
        ids: List[int] = []
        offsets = np.zeros(n + 1, dtype=np.int32)
        for i, p in enumerate(params):
            if p.filters():
                table[:, i] = (1.0, max(p.temperature, 0.0), math.log(p.min_p) if p.min_p > 0 else -math.inf,
                               p.top_k if 0 < p.top_k < V else 0, p.top_p, p.repetition_penalty)
                context = contexts[i]
                if abs(p.repetition_penalty - 1.0) >= 1.1920929e-07 and len(context):
                    win = (context if p.repeat_last_n == 0 or p.repeat_last_n >= len(context)
                           else context[-p.repeat_last_n:])
                    ids.extend(sorted({int(t) for t in win if 0 <= int(t) < V}))
            offsets[i + 1] = len(ids)
        dev = work.device
        pen_ids = torch.tensor(ids, dtype=torch.int32, device=dev) if ids else None
        hipops.filter_rows(work, torch.from_numpy(table).to(dev), pen_ids, torch.from_numpy(offsets).to(dev))

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], contexts: Sequence[Sequence[int]],
               rng_states: List[int]) -> List[int]:
        """One token per row of ``logits`` (fp32 ``[n, V]``).  ``rng_states[i]`` is advanced for
        every row that draws."""
        n = logits.shape[0]
        if n == 0:
            return []
        temps = np.zeros(n, dtype=np.float32)
        us = np.zeros(n, dtype=np.float32)
        work = logits
        if any(p.filters() for p in params):
            work = logits.clone()
            self._filter(work, params, contexts)
        for i, p in enumerate(params):
            if p.temperature > 0:
                temps[i] = 1.0 if p.filters() else p.temperature     # filtered rows are divided already
                rng_states[i], us[i] = lcg_next(rng_states[i])
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
        if temps.max() <= 0:
            if self._scratch is None or self._scratch[0].numel() < 32 * n:
                self._scratch = (torch.empty(32 * max(n, 64), dtype=torch.float32, device=logits.device),
                                 torch.empty(32 * max(n, 64), dtype=torch.int32, device=logits.device))
            hipops.argmax_rows(work, out, self._scratch[0], self._scratch[1], n)
        else:
            both = torch.from_numpy(np.stack([temps, us])).to(logits.device)
            hipops.sample_rows(work, both[0], both[1], out, n)
        return [int(x) for x in out.cpu().tolist()]
