"""Decode steps replayed from a HIP graph give the logits of the eager step, replay after
replay, with the program's own eager work (prefill steps of other shapes, new requests)
between the replays."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

CFG = dict(H.TINY_A, num_hidden_layers=4, hidden_size=128, num_attention_heads=4, num_key_value_heads=2, head_dim=64,
           intermediate_size=128, vocab_size=320)       # head size 64: the MFMA attention kernels run


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_graph_replays_equal_eager_steps(tmp_path, dtype):
    from spite_amd.engine.engine import Engine, StepEntry
    d = str(tmp_path / "m")
    H.make_model(d, CFG, seed=2, dtype=dtype)
    engines = [Engine(d, dtype=dtype, page_size=32, cache_tokens=1024, max_requests=4, graphs=g) for g in (True, False)]
    prompts = [H.random_tokens(CFG["vocab_size"], n, 20 + n) for n in (37, 5, 64)]
    late = H.random_tokens(CFG["vocab_size"], 45, 99)
    outs = []
    for eng in engines:
        rows = []
        slots = [eng.admit() for _ in prompts]
        logits = eng.step([StepEntry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
        toks = logits.argmax(-1).tolist()
        rows.append(logits.cpu().numpy().copy())
        for step in range(40):
            if step == 17:                      # eager work of another shape between replays
                slots.append(eng.admit())
                lg = eng.step([StepEntry(slots[-1], late, [len(late) - 1])])
                rows.append(lg.cpu().numpy().copy())
                toks.append(int(lg.argmax(-1)[0]))
            logits = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, toks)])
            toks = logits.argmax(-1).tolist()
            rows.append(logits.cpu().numpy().copy())
        outs.append(rows)
        eng.cache.check()
    assert engines[0].graph_replays >= 30 and engines[1].graph_replays == 0
    for a, b in zip(*outs):
        assert a.shape == b.shape and np.array_equal(a, b)


def test_a_graph_is_not_replayed_after_a_later_step_has_moved_the_workspaces(tmp_path):
    # a small decode shape is captured; the first decode step of a larger shape then grows the
    # scratch buffers (they start tiny here), which frees what the first graph points into; back
    # at the small shape the graph must be captured anew, not replayed
    from spite_amd.engine.engine import Engine, StepEntry
    d = str(tmp_path / "m")
    H.make_model(d, CFG, seed=4, dtype="bfloat16")
    prompts = [H.random_tokens(CFG["vocab_size"], 1 if i == 0 else 2, 70 + i) for i in range(7)]
    outs = []
    for graphs in (True, False):
        eng = Engine(d, dtype="bfloat16", page_size=32, cache_tokens=1024, max_requests=8, graphs=graphs,
                     workspace_bytes=1024)
        rows = []
        slots = [eng.admit()]
        tok = [int(eng.step([StepEntry(slots[0], prompts[0], [0])]).argmax(-1)[0])]
        for _ in range(6):                                   # seen, captured, replayed
            lg = eng.step([StepEntry(slots[0], [tok[0]], [0])])
            rows.append(lg.cpu().numpy().copy())
            tok = lg.argmax(-1).tolist()
        first = {k: v for k, v in eng._graphs.items() if v != "seen"}
        assert bool(first) == graphs
        for p in prompts[1:]:
            slots.append(eng.admit())
            tok.append(int(eng.step([StepEntry(slots[-1], p, [1])]).argmax(-1)[0]))
        before = eng._stamp()
        for _ in range(3):                                   # seven requests: seven rows of logits, more scratch
            lg = eng.step([StepEntry(s, [t], [0]) for s, t in zip(slots, tok)])
            rows.append(lg.cpu().numpy().copy())
            tok = lg.argmax(-1).tolist()
        if graphs:
            assert eng._stamp() != before, "the larger shape was meant to grow a workspace"
            assert all(eng._graphs.get(k) is not g for k, g in first.items()), "a stale graph was kept"
        for s in slots[1:]:
            eng.release(s)
        for _ in range(5):                                   # the small shape again
            lg = eng.step([StepEntry(slots[0], [tok[0]], [0])])
            rows.append(lg.cpu().numpy().copy())
            tok = [int(lg.argmax(-1)[0])]
        outs.append(rows)
        eng.cache.check()
    for a, b in zip(*outs):
        assert a.shape == b.shape and np.array_equal(a, b)


def test_a_capture_that_fails_midway_falls_back_to_eager_steps_with_the_right_logits():
    """A part that says it can be captured and cannot (it reads a value back on the host): the
    capture fails in the middle of the model.  What the recorded units took and handed on is put
    back, the step is finished eagerly with a warning, later steps run eagerly, and every logit
    equals the eager engine's."""
    import torch
    from spite_amd import Engine, StepEntry
    from spite_amd.parts import Mixer, ParamSpec, CacheNeed, register, PartSpec, BlockSpec, LayerCall, ModelSpec

    @register("mixer", "toy_claims_to_be_safe")
    class ClaimsToBeSafe(Mixer):
        graph_safe = True

        def __init__(self, env, width):
            self.width, self.w = width, None

        def params(self):
            return {"proj": ParamSpec((self.width, self.width))}

        def load(self, tensors):
            self.w = tensors["proj"]

        def cache_need(self):
            return CacheNeed()

        def forward(self, x, ctx, cache):
            gain = 1.0 + 0.0 * float(x[0, 0])              # a read-back: refused while a graph is recorded
            out = ctx.ws.take((ctx.T, self.width), torch.float32)
            torch.matmul(x.float() * gain, self.w.float().T, out=out)
            return out

    @register("mixer", "toy_reads_the_step_on_the_host")
    class ReadsTheHost(ClaimsToBeSafe):
        graph_safe = False

        def forward(self, x, ctx, cache):
            assert int(ctx.host.counts.sum()) == ctx.T           # the step's metadata, on the host
            out = ctx.ws.take((ctx.T, self.width), torch.float32)
            torch.matmul(x.float(), self.w.float().T, out=out)
            return out

    D, V = 32, 50
    g = torch.Generator().manual_seed(4)
    r = lambda *s: torch.randn(*s, generator=g) * 0.3
    norm = lambda name: PartSpec("rms", {"width": D, "eps": 1e-5}, {"weight": name})
    ffn = lambda p: PartSpec("dense_glu", {"hidden_size": D, "intermediate_size": 48}, {k: f"{p}.{k}" for k in ("gate_proj", "up_proj", "down_proj")})
    attn = lambda p: PartSpec("attention", dict(hidden_size=D, n_heads=2, n_kv_heads=1, head_dim=16,
                                                position=PartSpec("rotary", {"head_dim": 16, "theta": 100.0})),
                              {k: f"{p}.{k}" for k in ("q_proj", "k_proj", "v_proj", "o_proj")})
    # an honest eager unit first, so that the failing capture starts in the middle of the step
    blocks = [BlockSpec("prenorm", norm("b0.n1"), PartSpec("toy_reads_the_step_on_the_host", {"width": D}, {"proj": "b0.mix"}), norm("b0.n2"), ffn("b0.ffn")),
              BlockSpec("prenorm", norm("b1.n1"), PartSpec("toy_claims_to_be_safe", {"width": D}, {"proj": "b1.mix"}), norm("b1.n2"), ffn("b1.ffn")),
              BlockSpec("prenorm", norm("b2.n1"), attn("b2.attn"), norm("b2.n2"), ffn("b2.ffn"))]
    sp = ModelSpec("ToyFails", V, D, blocks, [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2)], norm("final"), "embed", "head")
    t = {"embed": r(V, D), "head": r(V, D), "final": 1 + r(D) * 0.1, "b1.mix": r(D, D), "b0.mix": r(D, D)}
    for b in range(3):
        t[f"b{b}.n1"], t[f"b{b}.n2"] = 1 + r(D) * 0.1, 1 + r(D) * 0.1
        t[f"b{b}.ffn.gate_proj"], t[f"b{b}.ffn.up_proj"], t[f"b{b}.ffn.down_proj"] = r(48, D), r(48, D), r(D, 48)
    for b in (2,):
        t[f"b{b}.attn.q_proj"], t[f"b{b}.attn.o_proj"] = r(32, D), r(D, 32)
        t[f"b{b}.attn.k_proj"], t[f"b{b}.attn.v_proj"] = r(16, D), r(16, D)
    outs = []
    for graphs in (True, False):
        eng = Engine(spec=sp, tensors=t, dtype="float32", page_size=4, cache_tokens=64, max_requests=2, graphs=graphs)
        assert [safe for _, _, safe in eng.model.graph_segments()] == [True, False, True]
        s = eng.admit()
        eng.step([StepEntry(s, [1, 2, 3], [])])
        rows = [eng.step([StepEntry(s, [4], [0])]).cpu().clone()]               # first decode step: eager
        if graphs:
            with pytest.warns(UserWarning, match="capturing"):
                rows.append(eng.step([StepEntry(s, [5], [0])]).cpu().clone())    # second: the capture fails midway
            assert not eng.use_graphs and eng.graph_replays == 0
        else:
            rows.append(eng.step([StepEntry(s, [5], [0])]).cpu().clone())
        rows += [eng.step([StepEntry(s, [6 + i], [0])]).cpu().clone() for i in range(4)]
        outs.append(rows)
    for a, b in zip(*outs):
        assert torch.equal(a, b)
