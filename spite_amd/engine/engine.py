"""The engine: a model on the GPU, its cache, and the one step function.

``Engine.step(entries)`` takes a batch of (request slot, its next tokens, wanted logit
places): portions of prompts beside single decoded tokens, cut anywhere.  It runs only the
tokens it is given, as one batch, against what earlier steps left in the cache, and returns
fp32 logits at the wanted places.  The reference's ``forward(tokens, logits_out, ctx)``
(crates/spite-models/src/lib.rs:330-335) is the one-request, every-position special case.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, Optional, Sequence, Union

import numpy as np
import torch

from ..cache.paged import PagedCache
from ..config import read_config
from ..csrc import hipops
from ..parts.base import ModelSpec, LayerCall, step_array_builder
from ..weights.loader import bind, FolderSource, DictSource, RandomSource
from .context import Env, Workspace, StepContext, LayerCache, HostBatch
from .model import Model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}
_CKPT_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


class EngineError(RuntimeError):
    pass


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()        # places among ``tokens`` whose logits are asked for


class StepMeta:
    """Metadata of one step: built on the host, sent to the GPU in one copy."""

    def __init__(self, engine: "Engine", entries: Sequence[StepEntry]):
        cache = engine.cache
        n = len(entries)
        slots = np.array([e.slot for e in entries], dtype=np.int32)
        counts = np.array([len(e.tokens) for e in entries], dtype=np.int32)
        starts = np.array([cache.cached(int(s)) for s in slots], dtype=np.int32)
        cu = np.zeros(n + 1, dtype=np.int32)
        np.cumsum(counts, out=cu[1:])
        T = int(cu[-1])
        n_groups = cache.n_groups()
        # table width: the next power of two, so that the shape of a step changes rarely
        widths = []
        for g in range(n_groups):
            w = max([cache.table_len(int(s), g) for s in slots], default=1)
            widths.append(max(4, 1 << (w - 1).bit_length()))
        self.widths = tuple(widths)
        rows = []
        for i, e in enumerate(entries):
            for w in e.want:
                if not 0 <= int(w) < counts[i]:
                    raise EngineError(f"entry {i}: wanted place {w} outside its {counts[i]} tokens")
                rows.append(int(cu[i]) + int(w))
        n_out = len(rows)
        # arrays that parts of this model derive from the batch (declared in ``step_arrays``)
        hb = HostBatch(slots=slots, starts=starts, counts=counts, cu_seqlens=cu)
        derived = {name: step_array_builder(name)(hb) for name in engine.model.step_arrays}
        # layout of the one int32 buffer
        sizes = [("token_ids", T), ("positions", T), ("seq_of_token", T), ("cu_seqlens", n + 1),
                 ("seq_slots", n), ("seq_starts", n), ("logit_rows", n_out)]
        sizes += [(f"derived:{name}", int(arr.size)) for name, (arr, _) in derived.items()]
        for g in range(n_groups):
            sizes += [(f"slot_map{g}", T), (f"table{g}", n * widths[g])]
        offs, total = {}, 0
        for name, sz in sizes:
            offs[name] = (total, sz)
            total += (sz + 63) // 64 * 64
        # where every array lies in the buffer: a captured step holds these addresses, so a step
        # may replay a graph only if its layout is the same (a part's derived array may change
        # its size between two steps of one shape)
        self.layout = tuple(o for o, _ in offs.values())
        host = engine._pinned(total)
        hv = {name: host[o:o + sz] for name, (o, sz) in offs.items()}
        tok = hv["token_ids"]
        for i, e in enumerate(entries):
            tok[cu[i]:cu[i + 1]] = np.asarray(e.tokens, dtype=np.int64)
        # position of token j of entry i: starts[i] + j
        hv["positions"][:] = np.arange(T, dtype=np.int32) + np.repeat(starts - cu[:-1], counts)
        hv["seq_of_token"][:] = np.repeat(np.arange(n, dtype=np.int32), counts)
        hv["cu_seqlens"][:] = cu
        for name, (arr, _) in derived.items():
            hv[f"derived:{name}"][:] = arr
        hv["seq_slots"][:] = slots
        hv["seq_starts"][:] = starts
        hv["logit_rows"][:] = np.asarray(rows, dtype=np.int32)
        for g in range(n_groups):
            cache.fill_step(slots, starts, counts, g, hv[f"slot_map{g}"], hv[f"table{g}"].reshape(n, widths[g]))
        dev = engine._upload(host, total)
        dv = {name: dev[o:o + sz] for name, (o, sz) in offs.items()}
        self.tables = [dv[f"table{g}"].view(n, widths[g]) for g in range(n_groups)]
        self.slot_maps = [dv[f"slot_map{g}"] for g in range(n_groups)]
        self.ctx = StepContext(
            T=T, n_seqs=n, token_ids=dv["token_ids"], positions=dv["positions"], seq_of_token=dv["seq_of_token"],
            cu_seqlens=dv["cu_seqlens"], seq_slots=dv["seq_slots"], seq_starts=dv["seq_starts"],
            logit_rows=dv["logit_rows"], n_out=n_out,
            host=hb, decode_only=bool(n > 0 and counts.max() == 1), max_count=int(counts.max()) if n else 0,
            derived={name: (dv[f"derived:{name}"], info) for name, (_, info) in derived.items()})
        self.host_tokens = tok[:T].copy()

    def layer_cache(self, cache: PagedCache, call: LayerCall):
        """The cache as the call's block sees it: one ``LayerCache``, or, for a block with several
        caches, a dict of them by the block's names."""
        def one(cid):
            state = cache.states.get(cid)
            if cid not in cache._group_of:
                return LayerCache(None, None, None, None, cache.page_size, call.write, state)
            g = cache.group_of(cid)
            k, v = cache.layer_pages(cid)
            return LayerCache(k, v, self.slot_maps[g], self.tables[g], cache.page_size, call.write, state,
                              cache.kv_tiled(cid))
        ids = call.cache_ids()
        return one(ids[""]) if set(ids) == {""} else {name: one(cid) for name, cid in ids.items()}


class Engine:
    def __init__(self, model: Union[str, dict, None] = None, *, dtype: str = "bfloat16", page_size: int = 64,
                 num_pages=None, cache_tokens: Optional[int] = None, max_batch_tokens: int = 2048,
                 max_requests: int = 8, device: str = "cuda:0", random_weights: bool = False, seed: int = 0,
                 init_std: float = 0.02, spec: Optional[ModelSpec] = None, tensors: Optional[dict] = None,
                 graphs: bool = True, workspace_bytes: int = 1 << 20):
        """``model``: a folder with config.json and model.safetensors; with ``random_weights`` a
        folder, a config.json path or a config dict whose weights are drawn on the GPU from
        ``seed``.  ``spec`` (+ ``tensors`` by checkpoint name, or ``random_weights``) builds a
        model from parts directly, without an architecture.  With ``graphs`` a decode step (one
        token of every request, every logit wanted) is captured in a HIP graph the second time
        its shape comes up and replayed from then on: the step is bound by kernel launches
        otherwise.  The graph holds the same kernels on the same buffers as the eager step.
        ``workspace_bytes``: the first size of the step's scratch buffers, which grow on demand."""
        if dtype not in _DTYPES:
            raise EngineError(f"dtype {dtype!r} (known: bfloat16, float32)")
        if not torch.cuda.is_available():
            raise EngineError("no GPU visible: the engine runs on the GPU only, there is no CPU path")
        hipops.lib()                      # fail now, loudly, when the kernels cannot be built or loaded
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.env = Env(_DTYPES[dtype], self.device)
        self.config = None
        ckpt_dtype = self.env.dtype
        if spec is None:
            if model is None:
                raise EngineError("Engine needs a model folder, a configuration or a spec")
            arch, self.config = read_config(model)
            spec = arch.build_spec(self.config)
            ckpt_dtype = _CKPT_DTYPES.get(getattr(self.config, "torch_dtype", "bfloat16"), torch.bfloat16)
        self.spec = spec
        self.model = Model(spec, self.env)
        self.page_size, self.max_batch_tokens, self.max_requests = int(page_size), int(max_batch_tokens), int(max_requests)
        # the cache first, in one piece per group, then the weights: the loaders' temporaries
        # (transposes, concatenations) must not cut the free memory into pieces before the
        # large pools are taken
        needs = self.model.cache_needs()
        if num_pages is None:
            tokens = cache_tokens if cache_tokens is not None else self.max_requests * 4096
            num_pages = max(1, -(-int(tokens) // self.page_size))
        self.cache = PagedCache(needs, self.page_size, num_pages, self.max_requests, self.env.dtype, self.device,
                                portion=self.max_batch_tokens)
        if tensors is not None:
            self._source = DictSource(tensors)
        elif random_weights:
            self._source = RandomSource(self.model.tensor_plan(), seed, init_std, ckpt_dtype)
        else:
            if not isinstance(model, str) or not os.path.isdir(model):
                raise EngineError("without random_weights the model must be a folder with model.safetensors")
            self._source = FolderSource(model, spec.strip_prefixes, spec.ignore_prefixes)
        bind(self.model, self._source, ckpt_dtype)
        torch.cuda.empty_cache()
        self.slow_paths = self._report_slow_paths()
        self._arenas = [Workspace(self.device, workspace_bytes), Workspace(self.device, workspace_bytes)]
        self._step_ws = Workspace(self.device, workspace_bytes)
        self._pin = None
        self._pin_event = None
        self._meta_dev = None
        self.steps_run = 0
        self.use_graphs = bool(graphs) and any(safe for _, _, safe in self.model.graph_segments())
        self._graphs: Dict[tuple, object] = {}     # shape of a decode step -> (segments, state), "seen" once, or "eager" for good
        self._graph_stamp = None
        self.graph_replays = 0

    def _report_slow_paths(self):
        """Says once, on standard error, which parts of this model will run a kernel far slower
        than the one meant for them, and why (a size one step off what the MFMA kernels take costs
        an order of magnitude, and nothing else would tell).  Returns {message: [blocks]}."""
        found: Dict[str, list] = {}
        if self.env.dtype != torch.bfloat16:
            return found
        for i, block in enumerate(self.model.blocks):
            for what, part, _ in block.children:
                for note in part.slow_paths(self.page_size):
                    found.setdefault(f"{what}: {note}", []).append(i)
        for what, part in (("embedding", self.model.embedding), ("head", self.model.head)):
            for note in part.slow_paths(self.page_size):
                found.setdefault(f"{what}: {note}", []).append(-1)
        if found:
            import sys
            for note, blocks in found.items():
                where = "" if blocks == [-1] else f" (blocks {blocks[0]}" + (f" to {blocks[-1]}, {len(blocks)} of them)" if len(blocks) > 1 else ")")
                print(f"[spite_amd] slow path: {note}{where}", file=sys.stderr, flush=True)
        return found

    # ------------------------------------------------------------------ weights
    def tensor_names(self):
        """Checkpoint names of the model's tensors, in the order of the layers."""
        return [f for f, _, _, _ in self.model.tensor_plan()]

    def get_tensor(self, name: str) -> torch.Tensor:
        """A tensor of the model by its checkpoint name, as its source stores it, on the host:
        read from the model folder, taken from the tensors given in memory, or drawn again from
        the seed (the same numbers as the GPU drew).  The parts keep their own layouts of it on
        the GPU (fused, transposed, in operand order)."""
        if name not in self._source.names():
            raise KeyError(f"{name!r} is not a tensor of {self._source.where}")
        return self._source.host(name)

    # ------------------------------------------------------------------ metadata transport
    def _pinned(self, n: int) -> np.ndarray:
        if self._pin_event is not None:
            self._pin_event.synchronize()
        if self._pin is None or self._pin.numel() < n:
            self._pin = torch.empty(max(n, 1 << 14), dtype=torch.int32, pin_memory=True)
            self._pin_np = self._pin.numpy()
        return self._pin_np

    def _upload(self, host: np.ndarray, n: int) -> torch.Tensor:
        if self._meta_dev is None or self._meta_dev.numel() < n:
            self._meta_dev = torch.empty(max(n, 1 << 14), dtype=torch.int32, device=self.device)
        self._meta_dev[:n].copy_(self._pin[:n], non_blocking=True)
        self._pin_event = torch.cuda.Event()
        self._pin_event.record()
        return self._meta_dev

    # ------------------------------------------------------------------ requests
    def admit(self) -> int:
        """A slot for a new request (its state is zeroed)."""
        return self.cache.admit()

    def release(self, slot: int) -> None:
        """The request is over: its pages and its slot are given back."""
        self.cache.release(slot)

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[StepEntry], commit: bool = True, trace: Optional[dict] = None) -> torch.Tensor:
        """Runs one batch; returns fp32 logits ``[wanted, vocab]`` on the GPU, in the order of
        the entries and of their ``want``.  Pages for the new positions are reserved here if
        the caller has not done so; with ``commit`` the positions count as cached afterwards
        and pages that no later query can read are given back.  ``trace``, a dict, is a
        testing aid: parts leave what they decided in it (``moe_experts``: one int32 tensor
        ``[tokens]`` per layer call with experts, in the order of the calls); a list under
        ``take_experts`` gives them the experts to take instead of their routers' choice."""
        if not entries:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        seen = set()
        V = self.spec.vocab_size
        total = 0
        for i, e in enumerate(entries):
            if e.slot in seen:
                raise EngineError(f"request slot {e.slot} appears twice in one step")
            seen.add(e.slot)
            if not self.cache.live(e.slot):
                raise EngineError(f"entry {i}: slot {e.slot} holds no request")
            if len(e.tokens) < 1:
                raise EngineError(f"entry {i}: no tokens")
            toks = np.asarray(e.tokens)
            if toks.min() < 0 or toks.max() >= V:
                bad = int(toks[(toks < 0) | (toks >= V)][0])
                raise EngineError(f"entry {i}: token id {bad} outside the vocabulary of {V}")
            total += len(e.tokens)
        self.cache.zero_fresh()       # state rows of slots handed out since the last step, by whomever
        self.cache.reserve_all([(e.slot, len(e.tokens)) for e in entries])    # every entry's pages, or nothing
        meta = StepMeta(self, entries)
        if trace is not None:
            meta.ctx.extras["trace"] = trace
        logits = None
        key = None
        if (self.use_graphs and trace is None and meta.ctx.decode_only and meta.ctx.n_out == meta.ctx.n_seqs
                and all(tuple(e.want) == (0,) for e in entries)):
            key = (meta.ctx.n_seqs, meta.widths, meta.layout)
            logits = self._replay(key, meta)
        if logits is None:
            self._step_ws.reset()
            if key is not None and self._graphs.get(key) == "seen":
                logits = self._capture(key, meta)
            else:
                logits = self.model.forward(meta.ctx, self.cache, meta, self._arenas, self._step_ws)
                if key is not None and key not in self._graphs:
                    self._graphs[key] = "seen"
                # this step may have grown a workspace (a first decode step of a larger shape
                # does): graphs captured before point into memory that the merge frees
                self._drop_stale_graphs()
        if commit:
            for e in entries:
                self.cache.commit(e.slot, len(e.tokens))
        self.steps_run += 1
        return logits

    # ------------------------------------------------------------------ graphs of decode steps
    def _stamp(self):
        """Changes whenever a buffer that graphs point into has been allocated anew."""
        return (self._meta_dev.data_ptr() if self._meta_dev is not None else 0, self._step_ws.generation,
                self._arenas[0].generation, self._arenas[1].generation)

    def _drop_stale_graphs(self) -> bool:
        """Forgets every captured graph if a buffer has moved since the stamp was taken (the
        marks of shapes seen once are no pointers and stay).  True if something moved."""
        stamp = self._stamp()
        if stamp == self._graph_stamp:
            return False
        self._graphs = {k: v for k, v in self._graphs.items() if isinstance(v, str)}
        self._graph_stamp = stamp
        return True

    # A captured step is a row of segments of the model's units: graphs over the runs of units
    # that can be captured, and between them the units that cannot (a part that reads the step's
    # metadata on the host), which run eagerly in every step on the buffers the graphs know.
    def _run_eager(self, lo, hi, state, meta):
        return self.model.run_units(lo, hi, state, meta.ctx, self.cache, meta, self._arenas, self._step_ws)

    @staticmethod
    def _addresses(state):
        return tuple((k, tuple(t.data_ptr() for t in (v if isinstance(v, tuple) else (v,)) if isinstance(t, torch.Tensor)))
                     for k, v in sorted(state.items()) if k != "logits")

    def _replay(self, key, meta):
        if self._drop_stale_graphs():
            return None
        hit = self._graphs.get(key)
        if hit is None or isinstance(hit, str):
            return None
        segments, state = hit
        for n, (lo, hi, graph, after) in enumerate(segments):
            if graph is not None:
                graph.replay()
                continue
            # the eager units of this step: the same buffers as in the captured step, or the rest
            # of the step runs eagerly too and the graphs are dropped
            live = dict(after["before"])
            for ws, mark in zip((*self._arenas, self._step_ws), after["marks"]):
                ws.rewind(mark)
            self._run_eager(lo, hi, live, meta)
            if self._stamp() != self._graph_stamp:
                self._graphs.pop(key, None)            # a buffer grew: captured anew when the shape comes up again
                self._drop_stale_graphs()
                return self._run_eager(hi, self.model.n_units(), live, meta)["logits"]
            if self._addresses(live) != after["addresses"]:
                # a part hands on memory of its own instead of the step's workspace: what follows
                # it cannot be replayed, so steps of this shape run eagerly from now on
                self._graphs[key] = "eager"
                return self._run_eager(hi, self.model.n_units(), live, meta)["logits"]
        self.graph_replays += 1
        return state["logits"]

    def _capture(self, key, meta):
        for ws in self._arenas:
            ws.reset()                     # merge what the warm-up step added, outside the capture
        self._drop_stale_graphs()          # the merge has freed what older graphs point into
        segments, state = [], {}
        for lo, hi, safe in self.model.graph_segments():
            if not safe:
                before, marks = dict(state), tuple(ws.mark() for ws in (*self._arenas, self._step_ws))
                self._run_eager(lo, hi, state, meta)
                segments.append((lo, hi, None, {"before": before, "marks": marks, "addresses": self._addresses(state)}))
                continue
            graph = torch.cuda.CUDAGraph()
            before, marks = dict(state), tuple(ws.mark() for ws in (*self._arenas, self._step_ws))
            try:
                with torch.cuda.graph(graph):
                    self._run_eager(lo, hi, state, meta)
            except Exception:
                # nothing of this segment has run yet (a capture computes nothing): what the units
                # took and handed on while they were recorded is put back, the rest of the step
                # runs eagerly, and so does every later step, loudly
                self._graphs.pop(key, None)
                self.use_graphs = False
                import warnings
                warnings.warn("capturing the decode step in a HIP graph failed; steps run eagerly from now on")
                for ws, mark in zip((*self._arenas, self._step_ws), marks):
                    ws.rewind(mark)
                return self._run_eager(lo, self.model.n_units(), before, meta)["logits"]
            if self._drop_stale_graphs():  # cannot happen (a workspace refuses to grow under capture)
                self._graphs.pop(key, None)
                return self._run_eager(lo, self.model.n_units(), state, meta)["logits"]
            graph.replay()                 # the capture itself computed nothing
            segments.append((lo, hi, graph, None))
        self._graphs[key] = (segments, state)
        self.graph_replays += 1
        return state["logits"]

    def commit(self, entries: Sequence[StepEntry]) -> None:
        for e in entries:
            self.cache.commit(e.slot, len(e.tokens))

    # ------------------------------------------------------------------ convenience
    def generate(self, prompts, max_tokens: int = 16, temperature: float = 0.0, seed: int = 0, **kw):
        from .generate import generate
        return generate(self, prompts, max_tokens=max_tokens, temperature=temperature, seed=seed, **kw)
