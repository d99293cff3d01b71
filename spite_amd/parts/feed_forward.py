"""Feed-forward parts.

``dense_glu`` (crates/spite-models/src/llama/llama4.rs:257-271):
y = W_down . (silu(W_gate . x) * (W_up . x)).

``moe_top1_sigmoid`` (crates/spite-models/src/moe.rs:87-194, llama4.rs:212-256): router
logits W_r . x in fp32; the expert with the largest logit (lowest index on ties); its
*input* is x * sigmoid(logit), its output is not weighted; a shared expert on the unscaled
x is added.  Routed and shared experts run as one grouped product over a row list: group
e < E holds the tokens routed to expert e, group E every token (at 33 to 64 tokens the shared
expert's group runs as a plain product of its own over the same rows).
"""
from __future__ import annotations

import math

import torch

from .base import FeedForward, ParamSpec, register
from .linear import SKINNY_MAX_ROWS, Weight, grouped_tile_shape, linear
from ..csrc import hipops


@register("ffn", "dense_glu")
class DenseGLU(FeedForward):
    graph_safe = True

    def __init__(self, env, hidden_size, intermediate_size):
        self.d, self.F = int(hidden_size), int(intermediate_size)
        self.w_gate_up = self.w_down = None

    def params(self):
        return {"gate_proj": ParamSpec((self.F, self.d)), "up_proj": ParamSpec((self.F, self.d)),
                "down_proj": ParamSpec((self.d, self.F))}

    def load(self, t):
        dt = t["gate_proj"].dtype if t["gate_proj"].dtype == t["up_proj"].dtype else torch.float32
        # gate rows then up rows: the up row of a gate row lies F rows further on; in operand order
        # that needs whole bands, F a multiple of 16
        self.w_gate_up = Weight(torch.cat([t["gate_proj"].to(dt), t["up_proj"].to(dt)], dim=0), self.F % 16 == 0)
        self.w_down = Weight(t["down_proj"])

    def slow_paths(self, page_size):
        return self.w_gate_up.slow_reason("gate/up projection") + self.w_down.slow_reason("down projection")

    def forward(self, x, x32, ctx, projected=None):
        T = x.shape[0]
        act = ctx.ws.take((T, self.F), x.dtype)
        linear(x, self.w_gate_up, act, glu=True, ws=ctx.ws)
        y = ctx.ws.take((T, self.d), torch.float32)
        linear(act, self.w_down, y, ws=ctx.ws)
        return (y,)


@register("ffn", "moe_top1_sigmoid")
class MoeTop1Sigmoid(FeedForward):
    graph_safe = True

    wants_f32_input = True

    def __init__(self, env, hidden_size, intermediate_size, n_experts, shared_intermediate_size=None):
        self.d, self.F, self.E = int(hidden_size), int(intermediate_size), int(n_experts)
        self.Fs = int(shared_intermediate_size if shared_intermediate_size is not None else intermediate_size)
        if self.E < 1 or self.E > 65000:
            raise ValueError(f"moe: {self.E} experts")
        self.fused_shared = self.Fs == self.F
        self.w_router = self.w_gate_up = self.w_down = None
        self.ws_gate_up = self.ws_down = None

    def params(self):
        d, F, Fs, E = self.d, self.F, self.Fs, self.E
        return {"router": ParamSpec((E, d), kind="vector"),
                "experts.gate_up_proj": ParamSpec((E, d, 2 * F)), "experts.down_proj": ParamSpec((E, F, d)),
                "shared.gate_proj": ParamSpec((Fs, d)), "shared.up_proj": ParamSpec((Fs, d)),
                "shared.down_proj": ParamSpec((d, Fs))}

    def load(self, t):
        self.w_router = t["router"].contiguous()
        # checkpoint [E, d, 2F] (x @ M) -> [E, 2F, d] rows of gate then up; down [E, F, d] -> [E, d, F]
        gu = t["experts.gate_up_proj"].transpose(1, 2)
        dn = t["experts.down_proj"].transpose(1, 2)
        sgu = torch.cat([t["shared.gate_proj"], t["shared.up_proj"]], dim=0)
        sdn = t["shared.down_proj"]
        if self.fused_shared and sgu.dtype == gu.dtype and sdn.dtype == dn.dtype:
            self.w_gate_up = Weight(torch.cat([gu, sgu[None]], dim=0), self.F % 16 == 0)
            self.w_down = Weight(torch.cat([dn, sdn[None]], dim=0))
        else:
            self.fused_shared = False
            self.w_gate_up, self.w_down = Weight(gu, self.F % 16 == 0), Weight(dn)
            self.ws_gate_up, self.ws_down = Weight(sgu, self.Fs % 16 == 0), Weight(sdn)

    def slow_paths(self, page_size):
        ws = [("experts' gate/up", self.w_gate_up), ("experts' down", self.w_down),
              ("shared expert's gate/up", self.ws_gate_up), ("shared expert's down", self.ws_down)]
        return [n for name, w in ws if w is not None for n in w.slow_reason(name)]

    def _few_rows_a_group(self, T: int) -> bool:
        """Whether a routed group of a step of T tokens is unlikely to hold more than 16 rows
        (group sizes taken as normal around T/E: mean + 4 sd)."""
        mean = T / self.E
        return mean + 4.0 * math.sqrt(T * (1.0 / self.E) * (1.0 - 1.0 / self.E)) <= 16.0

    def input_projection(self):
        return self.w_router if self.w_router is not None and self.w_router.dtype == torch.float32 else None

    def forward(self, x, x32, ctx, projected=None):
        """``projected``: the router's logits [T, E] if the block's norm formed them; else they
        are computed here from x32."""
        T, E, F, d = x.shape[0], self.E, self.F, self.d
        ws = ctx.ws
        expert = ws.take((T,), torch.int32)
        weight = ws.take((T,), torch.float32)
        trace = ctx.extras.get("trace")
        if trace is not None and trace.get("take_experts"):
            # a testing aid: the experts are given (one tensor per call, in the order of the
            # calls), each with the weight that its own logit gives; every other logit is
            # taken out before the plan is made
            take = trace["take_experts"].pop(0).to(device=x.device, dtype=torch.int64).view(T, 1)
            logits = projected
            if logits is None:
                logits = ws.take((T, E), torch.float32)
                hipops.gemm_generic(x32, self.w_router, logits, T, E, d)
            projected = torch.full_like(logits, float("-inf")).scatter_(1, take, logits.gather(1, take))
        if projected is None:
            hipops.router_top1(x32, self.w_router, expert, weight)
        n = 2 * T if self.fused_shared else T
        src, dst = ws.take((n,), torch.int32), ws.take((n,), torch.int32)
        scale = ws.take((n,), torch.float32)
        groups = E + 1 if self.fused_shared else E
        offsets = ws.take((groups + 1,), torch.int32)
        hipops.moe_plan(expert, weight, src, scale, dst, offsets, T, E, self.fused_shared, logits=projected)
        if trace is not None:                         # a testing aid: which expert each row took
            trace.setdefault("moe_experts", []).append(expert.clone())
        act = ws.take((n, F), x.dtype)
        y = ws.take((2 * T, d), torch.float32)
        if self.fused_shared and self.w_gate_up.tiled and 32 < T <= SKINNY_MAX_ROWS and self._few_rows_a_group(T):
            # 33 to 64 tokens: the routed groups hold a few rows each and take the weight stream's
            # narrow form (16 token columns); the shared expert, which takes every row, would be
            # read once per 16 of them there, so it runs as a plain product of its own (measured
            # at 64 tokens over 16 experts: 658 against 683 us for the two products of a layer)
            linear(x, self.w_gate_up, act, glu=True, offsets=offsets, n_groups=E, a_rows=src, a_scale=scale, rows=T,
                   max_rows=16, ws=ws)
            linear(x, self.w_gate_up.group(E), act[T:], glu=True, a_rows=src[T:], a_scale=scale[T:], rows=T, ws=ws)
            linear(act, self.w_down, y, offsets=offsets, n_groups=E, y_rows=dst, rows=T, max_rows=16, ws=ws)
            linear(act[T:], self.w_down.group(E), y, y_rows=dst[T:], rows=T, ws=ws)
            return (y[:T], y[T:])
        # the tile of either product, by the rounds that its tiles make on the chip (gate and up
        # rows share a tile of 512 W rows: 256 columns of the result; the down product's tile has 512)
        shape = grouped_tile_shape(T, E, groups - E, col_tiles=-(-F // 256)) if T > SKINNY_MAX_ROWS else 0
        shape_down = grouped_tile_shape(T, E, groups - E, col_tiles=-(-d // 512)) if T > SKINNY_MAX_ROWS else 0
        # every token goes to one expert: at most min(T, E) of their groups hold rows, and the shared one
        live = min(T, E) + (groups - E)
        linear(x, self.w_gate_up, act, glu=True, offsets=offsets, n_groups=groups, a_rows=src, a_scale=scale, rows=n,
               max_rows=T, tile_shape=shape, live_groups=live, ws=ws)
        # slot s writes row dst[s]: rows [0,T) the routed result per token, rows [T,2T) the shared one
        linear(act, self.w_down, y, offsets=offsets, n_groups=groups, y_rows=dst, rows=n, max_rows=T,
               tile_shape=shape_down, live_groups=live, ws=ws)
        if self.fused_shared:
            return (y[:T], y[T:])
        act_s = ws.take((T, self.Fs), x.dtype)
        linear(x, self.ws_gate_up, act_s, glu=True, ws=ws)
        linear(act_s, self.ws_down, y[T:], ws=ws)
        return (y[:T], y[T:])
