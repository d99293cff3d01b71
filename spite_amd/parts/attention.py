"""Grouped-query attention over the paged cache.

In order (crates/spite-models/src/llama/llama4.rs:130-207): fused q/k/v projection; position
encoding of q and k; the weightless RMS norm of every q and k head after the rotation
(:161-175) if ``qk_norm``; on layers with ``temperature`` the queries times
ln(floor((pos+1)/floor_scale)+1)*attn_scale+1 (:178-183); keys and values into the cache;
softmax(q.k/sqrt(hd)) over the keys that the layer's visibility allows
(crates/spite-compute/src/flash_attn.rs:71-158), head h on kv head h // (H/G); output
projection.  Scores, softmax and the output sum are fp32.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .base import Mixer, ParamSpec, CacheNeed, KVNeed, register, register_step_array, build as build_part
from .linear import linear, Weight
from ..csrc import hipops


def _tail_after_singles(host):
    """For a mixed step whose first entries hold one token each (decoded tokens lead, the
    scheduler's order): how many they are, and the running token counts of the entries behind
    them, from zero.  The decode kernel then takes the singles and the prefill kernel the rest;
    a query alone would fill a 256-column tile of the prefill kernel with a few columns."""
    counts, cu = host.counts, host.cu_seqlens
    n = len(counts)
    lead = 0
    while lead < n and counts[lead] == 1:
        lead += 1
    if lead == n or lead == 0:
        return np.zeros(0, dtype=np.int32), 0
    return (cu[lead:] - cu[lead]).astype(np.int32), lead


TAIL = "attention.tail_after_singles"
register_step_array(TAIL, _tail_after_singles)


@register("mixer", "attention")
class Attention(Mixer):
    graph_safe = True
    step_arrays = (TAIL,)

    def __init__(self, env, hidden_size, n_heads, n_kv_heads, head_dim, position, visibility="full", span=0,
                 qk_norm=False, qk_norm_eps=1e-5, temperature=None, softmax_scale=None, qk_norm_weighted=False,
                 qk_norm_first=False, score_cap=None):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads over {n_kv_heads} kv heads")
        if visibility not in hipops.VIS:
            raise ValueError(f"attention: visibility {visibility!r} (known: {sorted(hipops.VIS)})")
        if visibility != "full" and span < 1:
            raise ValueError(f"attention: {visibility} of size {span}")
        self.env = env
        self.d, self.H, self.G, self.hd = int(hidden_size), int(n_heads), int(n_kv_heads), int(head_dim)
        self.visibility, self.span = visibility, int(span or 0)
        # scaled scores capped smoothly before the softmax, cap * tanh(score / cap); None: no cap
        self.score_cap = float(score_cap or 0.0)
        if self.score_cap < 0:
            raise ValueError(f"attention: score cap {score_cap}")
        self.qk_norm, self.qk_norm_eps = bool(qk_norm), float(qk_norm_eps)
        # the head norm's weights ([hd] each for queries and keys) and its place: after the rotation
        # (Llama 4, weightless) or before it
        self.qk_norm_weighted, self.qk_norm_first = bool(qk_norm_weighted) and self.qk_norm, bool(qk_norm_first)
        self.w_qnorm = self.w_knorm = None
        self.temperature = temperature            # None or (floor_scale, attn_scale)
        self.scale = float(softmax_scale) if softmax_scale is not None else 1.0 / math.sqrt(self.hd)
        self.position = build_part("position", position, env)
        self.graph_safe = self.position.graph_safe
        self.wqkv = self.wo = self.slopes = None

    def params(self):
        d, H, G, hd = self.d, self.H, self.G, self.hd
        p = {"q_proj": ParamSpec((H * hd, d)), "k_proj": ParamSpec((G * hd, d)),
             "v_proj": ParamSpec((G * hd, d)), "o_proj": ParamSpec((d, H * hd))}
        if self.qk_norm_weighted:
            p["q_norm"] = ParamSpec((hd,), kind="vector", init="ones")
            p["k_norm"] = ParamSpec((hd,), kind="vector", init="ones")
        p.update({f"position.{k}": v for k, v in self.position.params().items()})
        return p

    def load(self, t):
        # one [(H+2G)*hd, d] operand: the reference splits a fused tensor the same way
        # (crates/spite-models/src/llama/llama4.rs:130-139)
        dts = {t[k].dtype for k in ("q_proj", "k_proj", "v_proj")}
        dt = torch.float32 if len(dts) > 1 else dts.pop()
        self.wqkv = Weight(torch.cat([t["q_proj"].to(dt), t["k_proj"].to(dt), t["v_proj"].to(dt)], dim=0))
        self.wo = Weight(t["o_proj"])
        if self.qk_norm_weighted:
            self.w_qnorm, self.w_knorm = t["q_norm"].contiguous(), t["k_norm"].contiguous()
        self.position.load({k[len("position."):]: v for k, v in t.items() if k.startswith("position.")})
        self.slopes = self.position.score_slopes(self.H)
        if self.slopes is not None and (self.slopes.dtype != torch.float32 or self.slopes.numel() != self.H):
            raise ValueError(f"attention: the position encoding's score slopes must be {self.H} fp32 values")

    def slow_paths(self, page_size):
        notes = []
        if self.env.dtype == torch.bfloat16:
            why = []
            if self.hd not in (64, 128):
                why.append(f"head size {self.hd} (the MFMA kernels have 64 and 128)")
            if page_size % 32:
                why.append(f"pages of {page_size} keys (they take multiples of 32)")
            if why:
                notes.append("attention runs on plain FMAs: " + ", ".join(why))
            for name, w in (("q/k/v projection", self.wqkv), ("output projection", self.wo)):
                if w is not None:
                    notes += w.slow_reason(name)
        return notes

    def cache_need(self):
        return CacheNeed(kv=KVNeed(self.G, self.hd, self.visibility, self.span))

    def _decode(self, q, o, ctx, cache, T):
        """The split-KV kernel over the step's first T tokens, each the only one of its request."""
        H, G, hd = self.H, self.G, self.hd
        # split the keys so that about two workgroups a compute unit run (measured: more splits
        # only add partial results to combine), each with at least eight blocks of keys; the
        # bound on the keys is the block table's width, so the launch is the same for every
        # step of that shape
        longest = cache.block_table.shape[1] * cache.page_size
        if self.visibility != "full":
            longest = min(longest, self.span + 32)
        blocks = -(-longest // 32)
        n_splits = max(1, min(-(-2 * hipops.cu_count() // (T * G)), -(-blocks // 8), 256))
        scratch = ctx.ws.take((hipops.attn_decode_workspace(T, H, hd, n_splits) // 4,), torch.float32)
        hipops.attn_decode(q, cache.k_pages, cache.v_pages, o, scratch, ctx.positions, ctx.seq_of_token,
                           cache.block_table, T, H, G, hd, cache.page_size, self.visibility, self.span,
                           self.scale, n_splits, softcap=self.score_cap, slopes=self.slopes)

    def _prefill(self, q, o, ctx, cache, lead, cu_seqlens):
        """The tiled kernel over the step's entries from ``lead`` on (portions of prompts)."""
        H, G, hd = self.H, self.G, self.hd
        counts, starts = ctx.host.counts[lead:], ctx.host.starts[lead:]
        # the most keys that a query of the step reads: what its request has cached, or no more than
        # the layer's span and the portion
        longest = int((starts + counts).max())
        if self.visibility != "full":
            longest = min(longest, self.span + int(counts.max()))
        n_splits = hipops.attn_prefill_splits(counts, H, G, longest)
        scratch = None
        if n_splits > 1:
            scratch = ctx.ws.take((hipops.attn_prefill_workspace(counts, H, G, hd, n_splits) // 4,), torch.float32)
        hipops.attn_prefill(q, cache.k_pages, cache.v_pages, o, ctx.positions[lead:], cu_seqlens, counts,
                            cache.block_table[lead:], H, G, hd, cache.page_size, self.visibility, self.span, self.scale,
                            n_splits=n_splits, scratch=scratch, softcap=self.score_cap, slopes=self.slopes)

    def forward(self, x, ctx, cache):
        T = x.shape[0]
        H, G, hd = self.H, self.G, self.hd
        ws = ctx.ws
        qkv = ws.take((T, (H + 2 * G) * hd), x.dtype)
        linear(x, self.wqkv, qkv, ws=ws)
        pe = self.position
        if not pe.fused:
            pe.transform(qkv, ctx.positions, H, G, hd)
        ka = pe.kernel_args() if pe.fused else {"use_rope": False, "inv_freq": None, "adjacent": False}
        q = ws.take((T, H * hd), x.dtype)
        temp = self.temperature
        hipops.rope_kvwrite(qkv, q, cache.k_pages, cache.v_pages, ctx.positions, cache.slot_map, ka["inv_freq"],
                            H, G, hd, cache.page_size, use_rope=ka["use_rope"], adjacent=ka["adjacent"],
                            use_norm=self.qk_norm, norm_eps=self.qk_norm_eps, use_temp=temp is not None,
                            floor_scale=temp[0] if temp else 1, attn_scale=temp[1] if temp else 0.0,
                            write_kv=cache.write, kv_tiled=cache.tiled, rotary_dim=ka.get("rotary_dim"),
                            norm_weight_q=self.w_qnorm, norm_weight_k=self.w_knorm, norm_first=self.qk_norm_first)
        o = ws.take((T, H * hd), x.dtype)
        # the MFMA kernels read pages in operand order (bfloat16, sizes in multiples of 32)
        mfma = cache.tiled and hd in (64, 128)
        if ctx.decode_only and mfma and H // G <= 16:
            self._decode(q, o, ctx, cache, T)
        elif mfma:
            cu_tail, lead = ctx.derived[TAIL]
            if lead and H // G <= 16:
                # decoded tokens of other requests beside prompt portions
                self._decode(q, o, ctx, cache, lead)
            else:
                lead = 0
            self._prefill(q[lead:], o[lead:], ctx, cache, lead, cu_tail if lead else ctx.cu_seqlens)
        else:
            hipops.attn_generic(q, cache.k_pages, cache.v_pages, o, ctx.positions, ctx.seq_of_token,
                                cache.block_table, T, H, G, hd, cache.page_size, self.visibility, self.span,
                                self.scale, kv_tiled=cache.tiled, softcap=self.score_cap, slopes=self.slopes)
        out = ws.take((T, self.d), torch.float32)
        linear(o, self.wo, out, ws=ws)
        return out
