"""A block of another arrangement, defined here: two mixers side by side, the built-in attention and
a toy attention over a narrow key (8 wide) and a wide value (24 wide), each with a cache of its own.
The block names its caches (`cache_needs`), the layer calls give every name a cache id, the cache
manager sizes the two halves of the toy's pool apart, and `forward` gets both caches by name.
Nothing of the framework's files changes."""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu
D, V, HEADS, KV, HD, KD, VD = 32, 40, 2, 1, 16, 8, 24


def define_parts():
    from spite_amd.parts import Block, Mixer, ParamSpec, CacheNeed, KVNeed, register, build

    @register("mixer", "toy_narrow_key")
    class NarrowKey(Mixer):
        """One head; keys 8 wide, values 24 wide, causal, no position encoding.  Its pages are
        read and written with plain tensor operations, request by request on the host."""

        def __init__(self, env, width):
            self.width, self.env = width, env

        def params(self):
            return {"q": ParamSpec((KD, self.width)), "k": ParamSpec((KD, self.width)), "v": ParamSpec((VD, self.width)),
                    "o": ParamSpec((self.width, VD))}

        def load(self, t):
            self.w = {k: v.float() for k, v in t.items()}

        def cache_need(self):
            return CacheNeed(kv=KVNeed(1, KD, "full", 0, v_head_dim=VD))

        def forward(self, x, ctx, cache):
            ps = cache.page_size
            assert cache.k_pages.shape[1:] == (1, ps, KD) and cache.v_pages.shape[1:] == (1, VD, ps) and not cache.tiled
            x = x.float()
            q, k, v = x @ self.w["q"].T, x @ self.w["k"].T, x @ self.w["v"].T
            rows = cache.slot_map.long()
            cache.k_pages[rows // ps, 0, rows % ps] = k.to(cache.k_pages.dtype)
            cache.v_pages[rows // ps, 0, :, rows % ps] = v.to(cache.v_pages.dtype)
            out = ctx.ws.take((ctx.T, self.width), torch.float32)
            cu = ctx.host.cu_seqlens
            for i in range(ctx.n_seqs):
                a, b, start = int(cu[i]), int(cu[i + 1]), int(ctx.host.starts[i])
                n = start + b - a
                pages = cache.block_table[i, :-(-n // ps)].long()
                keys = cache.k_pages[pages, 0].reshape(-1, KD)[:n].float()                       # [n, 8]
                vals = cache.v_pages[pages, 0].permute(0, 2, 1).reshape(-1, VD)[:n].float()      # [n, 24]
                score = q[a:b] @ keys.T / KD ** 0.5
                seen = torch.arange(n, device=x.device)[None, :] <= (start + torch.arange(b - a, device=x.device))[:, None]
                out[a:b] = torch.softmax(score.masked_fill(~seen, float("-inf")), -1) @ vals @ self.w["o"].T
            return out

    @register("block", "toy_two_mixers")
    class TwoMixers(Block):
        """h += attention(norm(h)) + narrow(norm(h)); h += ffn(norm2(h))."""

        def __init__(self, env, spec):
            self.env = env
            self.norm1, self.norm2 = build("norm", spec.norm1, env), build("norm", spec.norm2, env)
            self.attn, self.narrow = build("mixer", spec.mixer["attn"], env), build("mixer", spec.mixer["narrow"], env)
            self.ffn = build("ffn", spec.ffn, env)
            self.children = (("norm1", self.norm1, spec.norm1), ("attn", self.attn, spec.mixer["attn"]),
                             ("narrow", self.narrow, spec.mixer["narrow"]), ("norm2", self.norm2, spec.norm2),
                             ("ffn", self.ffn, spec.ffn))
            self.step_arrays = tuple(sorted({a for _, part, _ in self.children for a in part.step_arrays}))

        def cache_needs(self):
            return {"attn": self.attn.cache_need(), "narrow": self.narrow.cache_need()}

        def forward(self, h, pending, ctx, cache):
            n = ctx.ws.take(tuple(h.shape), self.env.dtype)
            self.norm1.forward(h, n, d1=pending[0] if len(pending) > 0 else None, d2=pending[1] if len(pending) > 1 else None)
            a = self.attn.forward(n, ctx, cache["attn"])
            b = self.narrow.forward(n, ctx, cache["narrow"])
            n2 = ctx.ws.take(tuple(h.shape), self.env.dtype)
            self.norm2.forward(h, n2, d1=a, d2=b)
            return tuple(self.ffn.forward(n2, None, ctx))


def spec():
    from spite_amd.parts import PartSpec, BlockSpec, LayerCall, ModelSpec
    norm = lambda name: PartSpec("rms", {"width": D, "eps": 1e-5}, {"weight": name})
    blocks = []
    for b in range(2):
        attn = PartSpec("attention", dict(hidden_size=D, n_heads=HEADS, n_kv_heads=KV, head_dim=HD,
                                          position=PartSpec("rotary", {"head_dim": HD, "theta": 100.0})),
                        {k: f"b{b}.attn.{k}" for k in ("q_proj", "k_proj", "v_proj", "o_proj")})
        narrow = PartSpec("toy_narrow_key", {"width": D}, {k: f"b{b}.narrow.{k}" for k in "qkvo"})
        ffn = PartSpec("dense_glu", {"hidden_size": D, "intermediate_size": 48},
                       {k: f"b{b}.ffn.{k}" for k in ("gate_proj", "up_proj", "down_proj")})
        blocks.append(BlockSpec("toy_two_mixers", norm(f"b{b}.n1"), {"attn": attn, "narrow": narrow}, norm(f"b{b}.n2"), ffn))
    order = [LayerCall(0, {"attn": 0, "narrow": 1}), LayerCall(1, {"attn": 2, "narrow": 3})]
    return ModelSpec("ToyTwoMixers", V, D, blocks, order, norm("final"), "embed", "head")


def tensors(seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.3
    t = {"embed": r(V, D), "head": r(V, D), "final": 1 + r(D) * 0.1}
    for b in range(2):
        t[f"b{b}.n1"], t[f"b{b}.n2"] = 1 + r(D) * 0.1, 1 + r(D) * 0.1
        t[f"b{b}.ffn.gate_proj"], t[f"b{b}.ffn.up_proj"], t[f"b{b}.ffn.down_proj"] = r(48, D), r(48, D), r(D, 48)
        t[f"b{b}.attn.q_proj"], t[f"b{b}.attn.o_proj"] = r(HEADS * HD, D), r(D, HEADS * HD)
        t[f"b{b}.attn.k_proj"], t[f"b{b}.attn.v_proj"] = r(KV * HD, D), r(KV * HD, D)
        t[f"b{b}.narrow.q"], t[f"b{b}.narrow.k"], t[f"b{b}.narrow.v"], t[f"b{b}.narrow.o"] = r(KD, D), r(KD, D), r(VD, D), r(D, VD)
    return t


def plain_model(t, tokens):
    import plain_llama4 as plain
    W = {k: v.double() for k, v in t.items()}
    T, pos = len(tokens), torch.arange(len(tokens))
    inv = plain.rope_inv_freq(HD, 100.0, None)
    mask = plain.visible_mask(pos, "full", 0)
    h = W["embed"][torch.tensor(tokens)]
    for b in range(2):
        n = plain.rms_norm(h, W[f"b{b}.n1"], 1e-5)
        q = plain.apply_rope((n @ W[f"b{b}.attn.q_proj"].T).view(T, HEADS, HD), pos, inv)
        k = plain.apply_rope((n @ W[f"b{b}.attn.k_proj"].T).view(T, KV, HD), pos, inv)
        v = (n @ W[f"b{b}.attn.v_proj"].T).view(T, KV, HD)
        a = plain.attention(q, k, v, mask).reshape(T, HEADS * HD) @ W[f"b{b}.attn.o_proj"].T
        score = (n @ W[f"b{b}.narrow.q"].T) @ (n @ W[f"b{b}.narrow.k"].T).T / KD ** 0.5
        nb = torch.softmax(score.masked_fill(~mask, float("-inf")), -1) @ (n @ W[f"b{b}.narrow.v"].T) @ W[f"b{b}.narrow.o"].T
        h = h + a + nb
        h = h + plain.swiglu_mlp(plain.rms_norm(h, W[f"b{b}.n2"], 1e-5), W[f"b{b}.ffn.gate_proj"], W[f"b{b}.ffn.up_proj"],
                                 W[f"b{b}.ffn.down_proj"])
    return (plain.rms_norm(h, W["final"], 1e-5) @ W["head"].T).float().numpy()


def test_a_block_with_two_mixers_and_caches_of_two_shapes():
    from spite_amd import Engine
    define_parts()
    t = tensors()
    eng = Engine(spec=spec(), tensors=t, dtype="float32", page_size=4, cache_tokens=96, max_requests=3)
    # two groups: the attention's pages and the toy's, whose keys and values have widths of their own
    shapes = sorted((tuple(g.k.shape[1:]), tuple(g.v.shape[1:])) for g in eng.cache.groups)
    assert shapes == [((24, 1, 4, KD), (24, 1, VD, 4)), ((24, 1, 4, HD), (24, 1, HD, 4))]
    assert all(g.k.shape[0] == 2 for g in eng.cache.groups)          # either group serves both blocks
    reqs = {"x": H.random_tokens(V, 23, 1), "y": H.random_tokens(V, 9, 2), "z": H.random_tokens(V, 15, 3)}
    ref = {(rid, i): row for rid, toks in reqs.items() for i, row in enumerate(plain_model(t, toks))}
    for steps in (H.schedule_whole(reqs), H.schedule_tail_one_by_one(reqs, tail=8),
                  H.schedule_portions(reqs, sizes=(3, 2, 7, 2)), H.schedule_mixed(reqs, seed=4, max_live=3)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), V)
        d, where = H.max_diff(got, ref)
        assert d < 1e-4, (d, where)


def test_a_layer_call_must_name_the_caches_its_block_has():
    from spite_amd import Engine
    from spite_amd.parts import LayerCall
    import dataclasses
    define_parts()
    bad = dataclasses.replace(spec(), order=[LayerCall(0, {"attn": 0}), LayerCall(1, {"attn": 1, "narrow": 2})])
    with pytest.raises(ValueError, match="caches"):
        Engine(spec=bad, tensors=tensors(), dtype="float32", page_size=4, cache_tokens=32, max_requests=2)
