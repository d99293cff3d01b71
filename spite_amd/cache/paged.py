"""The cache on the GPU: page pools per group of layers and per-request state tensors, with
the host-side bookkeeping in the native cache manager.

Layers are grouped by what they need: the same number of kv heads, head size and
visibility (every key, the query's chunk, a window).  A group's pool is two tensors, keys
``[layers, pages, kv_heads, page_size, key width]`` and values, transposed,
``[layers, pages, kv_heads, value width, page_size]`` (a mixer may ask for values of another
width than its keys); a page is the same row range in every layer of the group, so one block
table serves all of them.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..csrc import build, hostlib, hipops
from ..parts.base import CacheNeed

_KINDS = build.visibility_codes()     # "full", "chunk", "window": name -> code


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    pass


@dataclass
class Group:
    key: tuple                   # (kv heads, key width, visibility, span, value width)
    cache_ids: List[int]
    n_pages: int
    k: Optional[torch.Tensor] = None     # [layers, pages, G, page_size, key width]
    v: Optional[torch.Tensor] = None     # [layers, pages, G, value width, page_size]: values lie transposed

    def halves(self):
        """The pool's tensors (to fill or to poison all of it)."""
        return (self.k, self.v)


class PagedCache:
    def __init__(self, needs: Sequence[CacheNeed], page_size: int, num_pages, max_requests: int,
                 dtype: torch.dtype, device, allocate: bool = True, portion: Optional[int] = None):
        """``needs[i]``: what cache id i asks for.  ``num_pages``: pages of every group's pool
        (an int), or one number per group in order of first use.  With ``portion`` (the most
        tokens of one request in a step) and one number for all, a group whose layers read a
        chunk or a window only gets no more pages than ``max_requests`` requests can hold there
        at a time, each a chunk or window and a portion (``peak_pages``), however long they are."""
        self.page_size, self.max_requests, self.dtype, self.device = int(page_size), int(max_requests), dtype, device
        self.groups: List[Group] = []
        self._group_of: Dict[int, int] = {}
        self._layer_in_group: Dict[int, int] = {}
        by_key: Dict[tuple, int] = {}
        for cid, need in enumerate(needs):
            if need is None or need.kv is None:
                continue
            kv = need.kv
            key = (kv.n_kv_heads, kv.head_dim, kv.visibility, kv.span if kv.visibility != "full" else 0, kv.value_dim)
            if key not in by_key:
                by_key[key] = len(self.groups)
                self.groups.append(Group(key, [], 0, None))
            g = by_key[key]
            self._group_of[cid] = g
            self._layer_in_group[cid] = len(self.groups[g].cache_ids)
            self.groups[g].cache_ids.append(cid)
        n_groups = len(self.groups)
        pages = [int(num_pages)] * n_groups if isinstance(num_pages, int) else [int(x) for x in num_pages]
        if len(pages) != n_groups:
            raise CacheError(f"{len(pages)} pool sizes for {n_groups} groups")
        for g, n in zip(self.groups, pages):
            g.n_pages = n
        lib = hostlib.lib()
        self._lib = lib
        kinds = hostlib.int_array(_KINDS[g.key[2]] for g in self.groups)
        spans = hostlib.int_array(g.key[3] for g in self.groups)

        def create():
            h = lib.spc_create(self.page_size, self.max_requests, n_groups, kinds, spans, hostlib.int_array(pages))
            if not h:
                raise CacheError(hostlib.last_error())
            return h
        self._h = create()
        if portion is not None and isinstance(num_pages, int):
            cut = [min(n, self.max_requests * self.peak_pages(n * self.page_size, int(portion), g))
                   for g, n in enumerate(pages)]
            if cut != pages:
                lib.spc_destroy(self._h)
                pages = cut
                for g, n in zip(self.groups, pages):
                    g.n_pages = n
                self._h = create()
        self._fresh_buf = (ctypes.c_int * self.max_requests)()
        self.states: Dict[int, torch.Tensor] = {}
        if allocate:
            for g in self.groups:
                G, kd, vd = g.key[0], g.key[1], g.key[4]
                g.k = torch.zeros((len(g.cache_ids), g.n_pages, G, self.page_size, kd), dtype=dtype, device=device)
                g.v = torch.zeros((len(g.cache_ids), g.n_pages, G, vd, self.page_size), dtype=dtype, device=device)
            for cid, need in enumerate(needs):
                if need is not None and need.state is not None:
                    self.states[cid] = torch.zeros((self.max_requests, *need.state.shape),
                                                   dtype=need.state.dtype, device=device)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.spc_destroy(h)

    # ------------------------------------------------------------------ bookkeeping
    @property
    def handle(self):
        return self._h

    def n_groups(self):
        return len(self.groups)

    def group_of(self, cache_id: int) -> int:
        return self._group_of[cache_id]

    def admit(self) -> int:
        slot = self._lib.spc_admit(self._h)
        if slot < 0:
            raise CacheError(f"all {self.max_requests} request slots are taken")
        self.zero_fresh()
        return slot

    def zero_fresh(self) -> List[int]:
        """Clears the state rows of every slot that has been handed out since the last call, by
        whomever (this object's ``admit`` or the native scheduler, which admits on its own): the
        step function calls it before it runs, so a new request never meets the state that the
        slot's last request left.  Returns those slots."""
        # each slot is reported once however often it changed hands: never more than there are slots
        n = self._lib.spc_take_fresh(self._h, self._fresh_buf, len(self._fresh_buf))
        slots = list(self._fresh_buf[:n])
        if slots:
            for st in self.states.values():
                st[slots] = 0
        return slots

    def live(self, slot):
        return bool(self._lib.spc_live(self._h, slot))

    def cached(self, slot) -> int:
        return int(self._lib.spc_cached(self._h, slot))

    def can_reserve(self, slot, n) -> bool:
        return bool(self._lib.spc_can_reserve(self._h, slot, n))

    def reserve(self, slot, n):
        rc = self._lib.spc_reserve(self._h, slot, n)
        if rc == -1:
            raise OutOfPages(f"no pages for {n} more positions of slot {slot}: free "
                             f"{[self.free_pages(g) for g in range(self.n_groups())]}")
        if rc != 0:
            raise CacheError(f"reserve: slot {slot} is not live")

    def reserve_all(self, pairs):
        """``reserve`` for every ``(slot, n)`` of a step: all of them get their pages, or nothing
        changes and ``OutOfPages`` says so."""
        slots = (ctypes.c_int * max(len(pairs), 1))(*[int(s) for s, _ in pairs])
        counts = (ctypes.c_longlong * max(len(pairs), 1))(*[int(n) for _, n in pairs])
        rc = self._lib.spc_reserve_all(self._h, len(pairs), slots, counts)
        if rc == -1:
            raise OutOfPages(f"no pages for the step's {sum(n for _, n in pairs)} positions of slots "
                             f"{[s for s, _ in pairs]}: free {[self.free_pages(g) for g in range(self.n_groups())]}")
        if rc != 0:
            raise CacheError("reserve_all: a slot of the step is not live, or named twice")

    def commit(self, slot, n):
        rc = self._lib.spc_commit(self._h, slot, n)
        if rc != 0:
            raise CacheError(f"commit({slot}, {n}) failed with {rc}: not live, or more than was reserved")

    def release(self, slot):
        if self._lib.spc_release(self._h, slot) != 0:
            raise CacheError(f"release: slot {slot} is not live")

    def free_pages(self, g) -> int:
        return int(self._lib.spc_free_pages(self._h, g))

    def total_pages(self, g) -> int:
        return int(self._lib.spc_total_pages(self._h, g))

    def free_slots(self) -> int:
        return int(self._lib.spc_free_slots(self._h))

    def peak_pages(self, total, portion, g) -> int:
        return int(self._lib.spc_peak_pages(self._h, total, portion, g))

    def block_table(self, slot, g) -> List[int]:
        n = self._lib.spc_table_len(self._h, slot, g)
        if n < 0:
            raise CacheError(f"slot {slot} is not live")
        buf = (ctypes.c_int * max(n, 1))()
        self._lib.spc_table(self._h, slot, g, buf, n)
        return list(buf[:n])

    def check(self):
        if self._lib.spc_check(self._h) != 0:
            raise CacheError(hostlib.last_error())

    # ------------------------------------------------------------------ step metadata
    def fill_step(self, slots: np.ndarray, starts: np.ndarray, counts: np.ndarray, g,
                  slot_map_out: np.ndarray, table_out: np.ndarray):
        """Cache rows of every token of the step and one block-table row per entry (int32
        arrays, contiguous; one native call for the whole step)."""
        n, width = table_out.shape
        slots, starts, counts = (np.ascontiguousarray(a, dtype=np.int32) for a in (slots, starts, counts))
        if not (slot_map_out.dtype == table_out.dtype == np.int32 and slot_map_out.flags.c_contiguous
                and table_out.flags.c_contiguous and slot_map_out.size >= int(counts.sum()) and len(slots) == n):
            raise CacheError("fill_step: outputs must be contiguous int32 arrays of the step's sizes")
        rc = self._lib.spc_fill_step(self._h, n, slots.ctypes.data, starts.ctypes.data, counts.ctypes.data, g, width,
                                     slot_map_out.ctypes.data, table_out.ctypes.data)
        if rc == -4:
            raise CacheError("block table wider than planned")
        if rc != 0:
            raise CacheError("a slot of the step is not live")

    def table_len(self, slot, g) -> int:
        return int(self._lib.spc_table_len(self._h, slot, g))

    def kv_tiled(self, cache_id: int) -> bool:
        """Whether this cache's pages are kept in the MFMA attention kernels' operand order
        (bfloat16, head size and page size multiples of 32) rather than row-major."""
        g = self.groups[self._group_of[cache_id]]
        return g.key[1] == g.key[4] and hipops.kv_tiled_ok(self.dtype, g.key[1], self.page_size)

    def layer_pages(self, cache_id: int):
        g = self.groups[self._group_of[cache_id]]
        li = self._layer_in_group[cache_id]
        # keys [pages, G, page_size, key width]; values transposed: [pages, G, value width, page_size]
        return g.k[li], g.v[li]
