"""The framework takes parts it has never seen: a toy mixer with per-request state of fixed
size is defined here, registered, put into a model beside the built-in attention, and
stepped - whole, token by token and in portions, several requests in a batch - without a
change to the framework's files.  The layer order is data: one block runs twice (on caches
of its own), and one attention layer reads the cache that another layer wrote."""
import pytest
import torch

import helpers as H

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D, V, HEADS, KV, HD = 32, 50, 2, 1, 16


def define_parts():
    from spite_amd.parts import Mixer, ParamSpec, CacheNeed, StateNeed, register

    @register("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = W . mean(x_0..x_t): the state of a request is the sum of its inputs and their
        count, kept in the request's state slot between steps."""

        def __init__(self, env, width):
            self.width, self.env, self.w = width, env, None

        def params(self):
            return {"proj": ParamSpec((self.width, self.width))}

        def load(self, tensors):
            self.w = tensors["proj"]

        def cache_need(self):
            return CacheNeed(state=StateNeed((self.width + 1,), torch.float32))

        def forward(self, x, ctx, cache):
            out = ctx.ws.take((ctx.T, self.width), torch.float32)
            cu = ctx.host.cu_seqlens
            for i, slot in enumerate(ctx.host.slots):        # requests are walked on the host
                a, b = int(cu[i]), int(cu[i + 1])
                st = cache.state[int(slot)]
                sums = st[:self.width] + torch.cumsum(x[a:b].float(), 0)
                counts = st[self.width] + torch.arange(1, b - a + 1, device=x.device, dtype=torch.float32)
                mean = sums / counts[:, None]
                out[a:b] = mean @ self.w.float().T
                st[:self.width] = sums[-1]
                st[self.width] = counts[-1]
            return out


def spec(vis="window", span=6):
    from spite_amd.parts import PartSpec, BlockSpec, LayerCall, ModelSpec
    norm = lambda name: PartSpec("rms", {"width": D, "eps": 1e-5}, {"weight": name})
    ffn = lambda p: PartSpec("dense_glu", {"hidden_size": D, "intermediate_size": 48},
                             {k: f"{p}.{k}" for k in ("gate_proj", "up_proj", "down_proj")})
    attn = lambda p, vis, span: PartSpec(
        "attention", dict(hidden_size=D, n_heads=HEADS, n_kv_heads=KV, head_dim=HD, visibility=vis, span=span,
                          position=PartSpec("rotary", {"head_dim": HD, "theta": 100.0})),
        {k: f"{p}.{k}" for k in ("q_proj", "k_proj", "v_proj", "o_proj")})
    blocks = [
        BlockSpec("prenorm", norm("b0.n1"), PartSpec("toy_running_mean", {"width": D}, {"proj": "b0.mix"}), norm("b0.n2"), ffn("b0.ffn")),
        BlockSpec("prenorm", norm("b1.n1"), attn("b1.attn", vis, span), norm("b1.n2"), ffn("b1.ffn")),
        BlockSpec("prenorm", norm("b2.n1"), attn("b2.attn", vis, span), norm("b2.n2"), ffn("b2.ffn")),
    ]
    order = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 3),      # blocks 0 and 1 run twice
             LayerCall(2, 1, write=False)]                                             # block 2 reads cache 1
    return ModelSpec("ToyModel", V, D, blocks, order, norm("final"), "embed", "head")


def tensors(seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.3
    t = {"embed": r(V, D), "head": r(V, D), "final": 1 + r(D) * 0.1}
    for b in range(3):
        t[f"b{b}.n1"], t[f"b{b}.n2"] = 1 + r(D) * 0.1, 1 + r(D) * 0.1
        t[f"b{b}.ffn.gate_proj"], t[f"b{b}.ffn.up_proj"], t[f"b{b}.ffn.down_proj"] = r(48, D), r(48, D), r(D, 48)
    t["b0.mix"] = r(D, D)
    for b in (1, 2):
        t[f"b{b}.attn.q_proj"], t[f"b{b}.attn.o_proj"] = r(HEADS * HD, D), r(D, HEADS * HD)
        t[f"b{b}.attn.k_proj"], t[f"b{b}.attn.v_proj"] = r(KV * HD, D), r(KV * HD, D)
    return t


def plain_toy(t, tokens, vis="window", span=6):
    """The same model, whole sequence, in float64 torch."""
    import plain_llama4 as plain
    W = {k: v.double() for k, v in t.items()}
    T = len(tokens)
    pos = torch.arange(T)
    h = W["embed"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(HD, 100.0, None)
    mask = plain.visible_mask(pos, vis, span)
    kv = {}

    def ffn(b, x):
        return plain.swiglu_mlp(x, W[f"b{b}.ffn.gate_proj"], W[f"b{b}.ffn.up_proj"], W[f"b{b}.ffn.down_proj"])

    def attention(b, x, cache, write):
        q = plain.apply_rope((x @ W[f"b{b}.attn.q_proj"].T).view(T, HEADS, HD), pos, inv)
        if write:
            k = plain.apply_rope((x @ W[f"b{b}.attn.k_proj"].T).view(T, KV, HD), pos, inv)
            kv[cache] = (k, (x @ W[f"b{b}.attn.v_proj"].T).view(T, KV, HD))
        k, v = kv[cache]
        return plain.attention(q, k, v, mask).reshape(T, HEADS * HD) @ W[f"b{b}.attn.o_proj"].T

    for b, cache, write in ((0, 0, True), (1, 1, True), (0, 2, True), (1, 3, True), (2, 1, False)):
        n = plain.rms_norm(h, W[f"b{b}.n1"], 1e-5)
        if b == 0:
            mean = torch.cumsum(n, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
            h = h + mean @ W["b0.mix"].T
        else:
            h = h + attention(b, n, cache, write)
        h = h + ffn(b, plain.rms_norm(h, W[f"b{b}.n2"], 1e-5))
    return (plain.rms_norm(h, W["final"], 1e-5) @ W["head"].T).float().numpy()


def test_a_registered_toy_mixer_is_built_and_stepped():
    from spite_amd import Engine
    from spite_amd.parts import registered
    define_parts()
    assert "toy_running_mean" in registered("mixer")
    t = tensors()
    eng = Engine(spec=spec(), tensors=t, dtype="float32", page_size=4, cache_tokens=64, max_requests=3)
    # state slots only where the toy mixer runs; pages for the attention caches; cache 1 and 3 share a group
    assert sorted(eng.cache.states) == [0, 2] and eng.cache.n_groups() == 1
    assert eng.cache.states[0].shape == (3, D + 1)
    reqs = {"x": H.random_tokens(V, 23, 1), "y": H.random_tokens(V, 9, 2), "z": H.random_tokens(V, 15, 3)}
    ref = {(rid, i): row for rid, toks in reqs.items() for i, row in enumerate(plain_toy(t, toks))}
    for steps in (H.schedule_whole(reqs), H.schedule_tail_one_by_one(reqs, tail=8),
                  H.schedule_portions(reqs, sizes=(3, 2, 7, 2)), H.schedule_mixed(reqs, seed=4, max_live=3)):
        got = H.collect(steps, H.run_trace_inprocess(eng, steps), V)
        d, where = H.max_diff(got, ref)
        assert d < 1e-4, (d, where)
    # the window lets pages go while a request runs
    s = eng.admit()
    from spite_amd import StepEntry
    eng.step([StepEntry(s, reqs["x"], [])])
    assert eng.cache.block_table(s, 0)[:4] == [-1, -1, -1, -1]
    eng.release(s)


def test_an_unknown_part_or_a_bad_order_is_refused():
    from spite_amd import Engine
    from spite_amd.parts import PartSpec, LayerCall, UnknownPart
    define_parts()
    sp = spec()
    sp.blocks[0].mixer = PartSpec("no_such_mixer", {"width": D}, {"proj": "b0.mix"})
    with pytest.raises(UnknownPart, match="no_such_mixer"):
        Engine(spec=sp, tensors=tensors(), dtype="float32")
    sp = spec()
    sp.order = [LayerCall(2, 1, write=False)] + sp.order
    with pytest.raises(ValueError, match="before any call has written it"):
        Engine(spec=sp, tensors=tensors(), dtype="float32")
    sp = spec()
    sp.order.append(LayerCall(1, 1))
    with pytest.raises(ValueError, match="written by layer calls"):
        Engine(spec=sp, tensors=tensors(), dtype="float32")


def test_the_toy_mixer_is_served_by_generate_with_preemption_on_a_tiny_pool():
    # requests come and go through the native scheduler, which hands out slots on its own and
    # preempts when the pages run out: a request that gets a used slot, or is recomputed after a
    # preemption, must start from an empty state
    from spite_amd import Engine
    define_parts()
    t = tensors(5)
    # every key stays visible here, so that requests grow until the pages run out
    eng = Engine(spec=spec("full", 0), tensors=t, dtype="float32", page_size=4, num_pages=10, max_requests=3,
                 max_batch_tokens=12)
    prompts = [H.random_tokens(V, n, 30 + n) for n in (9, 14, 5, 11, 7, 3)]

    def plain_generate(p, n):
        toks = list(p)
        for _ in range(n):
            row = plain_toy(t, toks, "full", 0)[-1]
            toks.append(int(row.argmax()))
        return toks[len(p):]

    stats = {}
    got = eng.generate(prompts, max_tokens=7, temperature=0.0, eos_token_ids=[], stats=stats)
    assert stats["preemptions"] > 0, "the pool was meant to be too small for three requests at once"
    for p, g in zip(prompts, got):
        assert g == plain_generate(p, 7)
    eng.cache.check()


def test_graphs_hold_what_can_be_captured_around_a_mixer_that_cannot_be():
    """The toy mixer walks requests on the host, so it cannot be captured; the engine's graphs
    hold the units around it (embedding and first norm | feed-forward up to the next toy mixer's
    norm | the rest) and the mixer runs eagerly between them, on the buffers the graphs know.
    Same logits as eager steps, bit for bit, while requests come, go and take used slots."""
    from spite_amd import Engine, StepEntry
    define_parts()
    t = tensors(2)
    engines = [Engine(spec=spec("full", 0), tensors=t, dtype="float32", page_size=4, cache_tokens=400, max_requests=4, graphs=g)
               for g in (True, False)]
    assert engines[0].use_graphs and not engines[0].model.graph_safe
    kinds = [safe for _, _, safe in engines[0].model.graph_segments()]
    assert kinds == [True, False, True, False, True]
    prompts = [H.random_tokens(V, n, 70 + n) for n in (5, 9, 3, 7)]
    outs = []
    for eng in engines:
        rows, slots, last = [], {}, {}
        for i in (0, 1, 2):
            slots[i] = eng.admit()
            last[i] = int(eng.step([StepEntry(slots[i], prompts[i], [len(prompts[i]) - 1])])[0].argmax())
        for step in range(40):
            if step == 12:                   # one request ends, another takes its slot and its state rows
                eng.release(slots.pop(1))
                slots[3] = eng.admit()
                last[3] = int(eng.step([StepEntry(slots[3], prompts[3], [len(prompts[3]) - 1])])[0].argmax())
                del last[1]
            ids = sorted(slots)
            logits = eng.step([StepEntry(slots[i], [last[i]], [0]) for i in ids]).cpu()
            rows.append(logits.clone())
            for j, i in enumerate(ids):
                last[i] = int(logits[j].argmax())
        outs.append(rows)
    assert engines[0].graph_replays >= 30 and engines[1].graph_replays == 0
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # against the plain model: the first request's tokens, all forty of them
    toks = list(prompts[0])
    for step in range(40):
        row = plain_toy(t, toks, "full", 0)[-1] if step == 0 else ref
        toks.append(int(row.argmax()))
        ref = plain_toy(t, toks, "full", 0)[-1]
        assert abs(outs[0][step][0].numpy() - ref).max() < 1e-4, step


def test_a_part_that_hands_on_memory_of_its_own_keeps_its_steps_eager():
    """A mixer that returns a tensor of torch's instead of one from the step's workspace: what
    follows it cannot be replayed from a graph.  The engine notices at the first replay, finishes
    that step eagerly and runs steps of that shape eagerly from then on; the logits are right."""
    from spite_amd import Engine, StepEntry
    from spite_amd.parts import Mixer, ParamSpec, CacheNeed, register, PartSpec, BlockSpec, LayerCall, ModelSpec

    @register("mixer", "toy_own_memory")
    class OwnMemory(Mixer):
        def __init__(self, env, width):
            self.width, self.w = width, None

        def params(self):
            return {"proj": ParamSpec((self.width, self.width))}

        def load(self, tensors):
            self.w = tensors["proj"]

        def cache_need(self):
            return CacheNeed()

        def forward(self, x, ctx, cache):
            self.keep = getattr(self, "keep", []) + [torch.empty(64, device=x.device)]     # the allocator moves on
            return x.float() @ self.w.float().T

    norm = lambda name: PartSpec("rms", {"width": D, "eps": 1e-5}, {"weight": name})
    ffn = PartSpec("dense_glu", {"hidden_size": D, "intermediate_size": 48}, {k: f"b0.ffn.{k}" for k in ("gate_proj", "up_proj", "down_proj")})
    sp = ModelSpec("ToyOwn", V, D, [BlockSpec("prenorm", norm("b0.n1"), PartSpec("toy_own_memory", {"width": D}, {"proj": "b0.mix"}),
                                              norm("b0.n2"), ffn)], [LayerCall(0, 0)], norm("final"), "embed", "head")
    t = {k: v for k, v in tensors(3).items() if k in ("embed", "head", "final") or k.startswith("b0.")}
    outs = []
    for graphs in (True, False):
        eng = Engine(spec=sp, tensors=t, dtype="float32", page_size=4, cache_tokens=64, max_requests=2, graphs=graphs)
        s = eng.admit()
        eng.step([StepEntry(s, [1, 2, 3], [])])
        outs.append([eng.step([StepEntry(s, [4 + i], [0])]).cpu().clone() for i in range(8)])
        if graphs:
            assert "eager" in eng._graphs.values() and eng.graph_replays <= 1
    for a, b in zip(*outs):
        assert torch.equal(a, b)
