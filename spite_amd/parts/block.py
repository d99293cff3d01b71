"""Arrangement of a layer: pre-norm residual block,
h += mixer(norm1(h)); h += ffn(norm2(h)) (crates/spite-models/src/llama/llama4.rs:126-127,
202-211, 272-274).  The additions are folded into the norm that follows them: a block hands
its last increments to the next block (or the final norm) instead of adding them itself."""
from __future__ import annotations

import torch

from .base import Block, register, build as build_part, two_increments


@register("block", "prenorm")
class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, env, spec):
        self.env = env
        self.norm1 = build_part("norm", spec.norm1, env)
        self.mixer = build_part("mixer", spec.mixer, env)
        self.norm2 = build_part("norm", spec.norm2, env)
        self.ffn = build_part("ffn", spec.ffn, env)
        self.children = (("norm1", self.norm1, spec.norm1), ("mixer", self.mixer, spec.mixer),
                         ("norm2", self.norm2, spec.norm2), ("ffn", self.ffn, spec.ffn))
        self.graph_safe = all(part.graph_safe for _, part, _ in self.children)
        self.step_arrays = tuple(sorted({a for _, part, _ in self.children for a in part.step_arrays}))

    def forward(self, h, pending, ctx, cache):
        state = {"h": h, "pending": pending}
        for _, stage in self.stages():
            stage(state, ctx, cache)
        return state["pending"]

    def stages(self):
        # first norm | mixer | second norm and feed-forward: a mixer that reads the step's metadata
        # on the host keeps only itself out of a graph
        return [(self.norm1.graph_safe, self._stage_norm1), (self.mixer.graph_safe, self._stage_mixer),
                (self.norm2.graph_safe and self.ffn.graph_safe, self._stage_ffn)]

    def _stage_norm1(self, state, ctx, cache):
        h = state["h"]
        d1, d2 = two_increments(h, state["pending"])
        n = ctx.ws.take(tuple(h.shape), self.env.dtype)
        self.norm1.forward(h, n, d1=d1, d2=d2)
        state["normed"] = n

    def _stage_mixer(self, state, ctx, cache):
        state["mixed"] = self.mixer.forward(state.pop("normed"), ctx, cache)

    def _stage_ffn(self, state, ctx, cache):
        h, delta, ws = state["h"], state.pop("mixed"), ctx.ws
        T, d = h.shape
        n2 = ws.take((T, d), self.env.dtype)
        proj = self.ffn.input_projection()
        if proj is not None and self.norm2.can_project(proj):
            # the norm forms the feed-forward's small fp32 products (router logits) itself
            logits = ws.take((T, proj.shape[0]), torch.float32)
            self.norm2.forward(h, n2, d1=delta, proj=proj, proj_out=logits)
            state["pending"] = tuple(self.ffn.forward(n2, None, ctx, projected=logits))
            return
        n2_32 = None
        if self.ffn.wants_f32_input:
            n2_32 = n2 if n2.dtype == torch.float32 else ws.take((T, d), torch.float32)
        self.norm2.forward(h, n2, d1=delta, out32=None if n2_32 is n2 else n2_32)
        state["pending"] = tuple(self.ffn.forward(n2, n2_32, ctx))
