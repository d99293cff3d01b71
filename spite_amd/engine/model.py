"""A model: blocks built from a ``ModelSpec``, the order in which they run, embedding and
output matrix.  The same class serves every architecture; what differs is the spec."""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..csrc import hipops
from ..parts import base as P
from ..parts.base import ParamSpec, PartSpec, CacheNeed
from .context import Env, Workspace, StepContext


class Model:
    def __init__(self, spec: P.ModelSpec, env: Env):
        self.spec, self.env = spec, env
        self.blocks = [P.build("block", PartSpec(bs.kind, {"spec": bs}), env) for bs in spec.blocks]
        self.final_norm = P.build("norm", spec.final_norm, env)
        V, d = spec.vocab_size, spec.hidden_size
        self.embedding_spec = spec.embedding or PartSpec("token_table", {"vocab_size": V, "width": d},
                                                         {"weight": spec.embed_name})
        self.head_spec = spec.head or PartSpec("linear_head", {"vocab_size": V, "width": d, "tied": spec.head_name is None},
                                               {} if spec.head_name is None else {"weight": spec.head_name})
        if spec.embedding is None and spec.embed_name is None:
            raise ValueError("the model spec names neither an embedding part nor the embedding table's tensor")
        self.embedding = P.build("embedding", self.embedding_spec, env)
        self.head = P.build("head", self.head_spec, env)
        for i, call in enumerate(spec.order):
            if not 0 <= call.block < len(self.blocks):
                raise ValueError(f"layer call {i} names block {call.block} of {len(self.blocks)}")
            wanted, given = set(self.blocks[call.block].cache_needs()), set(call.cache_ids())
            if wanted != given and not (len(wanted) == 1 and given == {""}):
                raise ValueError(f"layer call {i}: block {call.block} has the caches {sorted(wanted)}, the call names {sorted(given)}")
        writers = {}
        for i, call in enumerate(spec.order):
            if call.write:
                for cid in call.cache_ids().values():
                    if cid in writers:
                        raise ValueError(f"cache {cid} is written by layer calls {writers[cid]} and {i}")
                    writers[cid] = i
        for i, call in enumerate(spec.order):
            for cid in call.cache_ids().values():
                if not call.write and (cid not in writers or writers[cid] > i):
                    raise ValueError(f"layer call {i} reads cache {cid} before any call has written it")
        self._writers = writers
        self._units = self._build_units()
        self.graph_safe = all(u[1] for u in self._units)
        self.step_arrays = tuple(sorted({a for b in self.blocks for a in b.step_arrays}))

    # ------------------------------------------------------------------ tensors
    def tensor_plan(self) -> List[Tuple[str, ParamSpec, object, str]]:
        """(checkpoint name, spec, owning part, local name) of every tensor of the model."""
        plan = []
        ends = [("embedding", self.embedding, self.embedding_spec), ("head", self.head, self.head_spec)]
        for what, part, pspec in ends:
            for local, ps in part.params().items():
                if local not in pspec.names or pspec.names[local] is None:
                    raise KeyError(f"the {what} {pspec.kind!r} declares tensor {local!r} but its spec names no "
                                   f"checkpoint tensor for it")
                plan.append((pspec.names[local], ps, part, local))
        for local, ps in self.final_norm.params().items():
            plan.append((self.spec.final_norm.names[local], ps, self.final_norm, local))
        for block in self.blocks:
            for _, part, pspec in block.children:
                for local, ps in part.params().items():
                    if local not in pspec.names:
                        raise KeyError(f"part {pspec.kind!r} declares tensor {local!r} but its spec names no "
                                       f"checkpoint tensor for it")
                    plan.append((pspec.names[local], ps, part, local))
        return plan

    def finish_loading(self):
        self.head.tie(self.embedding)

    def cache_needs(self) -> List[Optional[CacheNeed]]:
        """What every cache id asks for: what the block of the call that writes it says."""
        n = max((cid for c in self.spec.order for cid in c.cache_ids().values()), default=-1) + 1
        needs: List[Optional[CacheNeed]] = [None] * n
        for cid, i in self._writers.items():
            call = self.spec.order[i]
            of_block = self.blocks[call.block].cache_needs()
            for name, c in call.cache_ids().items():
                if c == cid:
                    needs[cid] = of_block[name] if name in of_block else next(iter(of_block.values()))
        return needs

    # ------------------------------------------------------------------ one step
    # A step is a row of units: the embedding, every layer call, and the tail (final norm and
    # head).  ``forward`` runs them all; the engine's graphs run them in segments, so that a part
    # that cannot be captured costs an eager call of its own unit and nothing else.
    def _build_units(self):
        units = [("embed", self.embedding.graph_safe, None, None)]
        for i, call in enumerate(self.spec.order):
            for j, (safe, fn) in enumerate(self.blocks[call.block].stages()):
                units.append(("stage", bool(safe), i, (j, fn)))
        units.append(("tail", self.final_norm.graph_safe and self.head.graph_safe, None, None))
        return units

    def n_units(self) -> int:
        return len(self._units)

    def graph_segments(self) -> List[Tuple[int, int, bool]]:
        """Maximal runs of units ``(first, end, safe)`` that can (or cannot) be captured."""
        segs, lo, units = [], 0, self._units
        for u in range(1, len(units) + 1):
            if u == len(units) or units[u][1] != units[lo][1]:
                segs.append((lo, u, units[lo][1]))
                lo = u
        return segs

    def run_units(self, lo: int, hi: int, state: dict, ctx: StepContext, cache, meta, arenas, step_ws: Workspace) -> dict:
        """Runs units ``lo .. hi-1``.  ``state`` carries the residual stream ``h``, the increments
        that the next norm has to add (``pending``), what a block's stages hand each other and,
        after the tail, ``logits``."""
        n, d = len(self.spec.order), self.spec.hidden_size
        for u in range(lo, hi):
            kind, _, i, stage = self._units[u]
            if kind == "embed":
                state["h"] = step_ws.take((ctx.T, d), torch.float32)
                state["pending"] = ()
                ctx.ws = arenas[0]
                self.embedding.forward(ctx.token_ids, state["h"], ctx)
            elif kind == "stage":
                ctx.ws = arenas[i % 2]
                if stage[0] == 0:
                    ctx.ws.reset()
                stage[1](state, ctx, meta.layer_cache(cache, self.spec.order[i]))
            else:
                ctx.ws = arenas[n % 2]
                ctx.ws.reset()
                if ctx.n_out == 0:
                    state["logits"] = torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.env.device)
                    continue
                d1, d2 = P.two_increments(state["h"], state["pending"])
                rows = ctx.ws.take((ctx.n_out, d), self.env.dtype)
                self.final_norm.forward(state["h"], rows, d1=d1, d2=d2, rows=ctx.logit_rows, write_h=False)
                state["logits"] = step_ws.take((ctx.n_out, self.spec.vocab_size), torch.float32)
                self.head.forward(rows, state["logits"], ctx)
        return state

    def forward(self, ctx: StepContext, cache, meta, arenas, step_ws: Workspace) -> torch.Tensor:
        """Runs the tokens of the step through every layer call; returns fp32 logits
        ``[n_out, V]`` at ``ctx.logit_rows``."""
        return self.run_units(0, self.n_units(), {}, ctx, cache, meta, arenas, step_ws)["logits"]
