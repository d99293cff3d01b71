"""Python face of the native scheduler (``csrc/host/scheduler.h``).  Names after the
reference's crates/spite-scheduler/src/lib.rs:55-92."""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import List, Sequence


from ..csrc import hostlib

FINISH_REASONS = ("NotDone", "EosToken", "StopToken", "MaxTokens", "ContextLimit", "OutOfPages", "Cancelled")
SLOT_STATES = ("Free", "Prefilling", "Generating", "Done")


class SchedulerError(RuntimeError):
    pass


@dataclass
class BatchEntry:
    request_id: int
    slot: int
    start: int
    tokens: List[int]
    wants_logits: bool


@dataclass
class BatchOutput:
    request_id: int
    token: int            # -1: nothing emitted
    done: bool
    finish_reason: str


class Scheduler:
    def __init__(self, cache, max_batch_tokens: int, max_context: int, eos_tokens: Sequence[int] = ()):
        self._lib = hostlib.lib()
        self._cache = cache              # keeps the native manager alive
        eos = hostlib.int_array(eos_tokens)
        self._h = self._lib.sps_create(cache.handle, int(max_batch_tokens), int(max_context), eos, len(list(eos_tokens)))
        if not self._h:
            raise SchedulerError(hostlib.last_error())
        self.max_batch_tokens = int(max_batch_tokens)
        cap = cache.max_requests + 1
        self._ids = (ctypes.c_ulonglong * cap)()
        self._slots = (ctypes.c_int * cap)()
        self._starts = (ctypes.c_longlong * cap)()
        self._counts = (ctypes.c_int * cap)()
        self._wants = (ctypes.c_int * cap)()
        self._tokens = (ctypes.c_int * (self.max_batch_tokens + 1))()
        self._cap = cap

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.sps_destroy(h)

    def submit(self, prompt: Sequence[int], max_tokens: int, stop_tokens: Sequence[int] = ()) -> int:
        p = hostlib.int_array(prompt)
        s = hostlib.int_array(stop_tokens)
        rid = self._lib.sps_submit(self._h, p, len(prompt), int(max_tokens), s, len(stop_tokens))
        if rid == 0:
            raise SchedulerError(hostlib.last_error())
        return int(rid)

    def schedule(self) -> List[BatchEntry]:
        ntok = ctypes.c_int(0)
        n = self._lib.sps_schedule(self._h, self._cap, self.max_batch_tokens, self._ids, self._slots, self._starts,
                                   self._counts, self._wants, self._tokens, ctypes.byref(ntok))
        if n < 0:
            raise SchedulerError(hostlib.last_error())
        out, off = [], 0
        for i in range(n):
            c = self._counts[i]
            out.append(BatchEntry(int(self._ids[i]), self._slots[i], int(self._starts[i]),
                                  list(self._tokens[off:off + c]), bool(self._wants[i])))
            off += c
        return out

    def update(self, sampled: Sequence[int]) -> List[BatchOutput]:
        s = hostlib.int_array(sampled)
        cap = self._cap + 8
        ids = (ctypes.c_ulonglong * cap)()
        toks = (ctypes.c_int * cap)()
        done = (ctypes.c_int * cap)()
        why = (ctypes.c_int * cap)()
        n = self._lib.sps_update(self._h, s, len(sampled), cap, ids, toks, done, why)
        if n < 0:
            raise SchedulerError(hostlib.last_error())
        return [BatchOutput(int(ids[i]), toks[i], bool(done[i]), FINISH_REASONS[why[i]]) for i in range(n)]

    def cancel(self, request_id: int) -> bool:
        return bool(self._lib.sps_cancel(self._h, request_id))

    @property
    def n_waiting(self):
        return self._lib.sps_n_waiting(self._h)

    @property
    def n_running(self):
        return self._lib.sps_n_running(self._h)

    def active_count(self):
        return self.n_waiting + self.n_running

    @property
    def n_preemptions(self):
        return int(self._lib.sps_n_preemptions(self._h))

    def request_info(self, request_id: int):
        buf = (ctypes.c_longlong * 5)()
        if self._lib.sps_request_info(self._h, request_id, buf) != 0:
            return None
        return {"state": SLOT_STATES[buf[0]], "slot": int(buf[1]), "n_computed": int(buf[2]),
                "n_generated": int(buf[3]), "n_preempted": int(buf[4])}
