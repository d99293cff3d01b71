"""Each part alone: the part objects that the engine built for a tiny model are fed made-up
activations, outside any model, and compared with the plain implementation's function for
that part.  Mixers are stepped twice on one request (a portion, then another) so that the
second call reads what the first left in the cache."""

import numpy as np
import pytest
import torch

import helpers as H
import plain_llama4 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class Rig:
    def __init__(self, name, dtype, tmp):
        from spite_amd import Engine
        self.cfg = H.CONFIGS[name]
        self.dir = str(tmp / f"{name}_{dtype}")
        self.w = H.make_model(self.dir, self.cfg, seed=21, dtype=dtype)
        self.eng = Engine(self.dir, dtype=dtype, page_size=8, cache_tokens=512, max_requests=4)
        self.dt = self.eng.env.dtype
        self.tol = 3e-5 if dtype == "float32" else 2.5e-2
        self.d = self.cfg["hidden_size"]

    def context(self, entries):
        """A step's context for [(slot, n_tokens)], with pages reserved; and the workspace."""
        from spite_amd.engine.engine import StepMeta, StepEntry
        from spite_amd.engine.context import Workspace
        es = [StepEntry(s, [0] * n, []) for s, n in entries]
        for e in es:
            self.eng.cache.reserve(e.slot, len(e.tokens))
        meta = StepMeta(self.eng, es)
        meta.ctx.ws = Workspace(self.eng.device, 1 << 22)
        return meta

    def commit(self, entries):
        for s, n in entries:
            self.eng.cache.commit(s, n)

    def acts(self, T, seed, scale=1.0):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(T, self.d, generator=g) * scale
        return x.to(self.dt).to(DEV), x.to(self.dt).double()      # what the part gets, and the same numbers for the plain side

    def close(self, got, ref, what):
        err = (got.double().cpu() - ref).abs().max().item()
        scale = max(ref.abs().max().item(), 1e-3)
        assert err <= self.tol * scale, f"{what}: {err} against a scale of {scale}"


@pytest.fixture(scope="module", params=[("A", "float32"), ("B", "float32"), ("A", "bfloat16"), ("B", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def rig(request, tmp_path_factory):
    return Rig(*request.param, tmp_path_factory.mktemp("parts"))


def test_norm_alone(rig):
    blk = rig.eng.model.blocks[1]
    T, d = 6, rig.d
    g = torch.Generator().manual_seed(1)
    h, d1, d2 = (torch.randn(T, d, generator=g) for _ in range(3))
    out = torch.empty(T, d, dtype=rig.dt, device=DEV)
    out32 = torch.empty(T, d, dtype=torch.float32, device=DEV)
    hh = h.to(DEV)
    blk.norm2.forward(hh, out, d1=d1.to(DEV), d2=d2.to(DEV), out32=out32)
    w = rig.w["model.layers.1.post_attention_layernorm.weight"]
    ref = plain.rms_norm((h + d1 + d2).double(), w, rig.cfg["rms_norm_eps"])
    rig.close(out, ref, "norm")
    assert (out32.double().cpu() - ref).abs().max() < 3e-5 * ref.abs().max()
    assert (hh.cpu().double() - (h + d1 + d2).double()).abs().max() < 1e-6       # the sum is kept in the stream


def test_position_encoding_alone(rig):
    cfg = rig.cfg
    hd = cfg["head_dim"]
    rot = rig.eng.model.blocks[0].mixer.position
    nope = rig.eng.model.blocks[3].mixer.position
    ref = plain.rope_inv_freq(hd, cfg["rope_theta"], cfg["rope_scaling"])
    assert torch.allclose(rot.kernel_args()["inv_freq"].cpu().double(), ref, rtol=1e-6)
    assert rot.kernel_args()["use_rope"] and not nope.kernel_args()["use_rope"]


def plain_mixer(rig, L, x, positions):
    """The plain implementation's attention sub-layer on whole sequences (positions from 0)."""
    cfg, W = rig.cfg, rig.w
    H_, G, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    p = f"model.layers.{L}.self_attn."
    T = x.shape[0]
    q = (x @ W[p + "q_proj.weight"].T).view(T, H_, hd)
    k = (x @ W[p + "k_proj.weight"].T).view(T, G, hd)
    v = (x @ W[p + "v_proj.weight"].T).view(T, G, hd)
    rope, _ = plain.layer_kinds(cfg)
    if rope[L]:
        inv = plain.rope_inv_freq(hd, cfg["rope_theta"], cfg["rope_scaling"])
        q, k = plain.apply_rope(q, positions, inv), plain.apply_rope(k, positions, inv)
        if cfg["use_qk_norm"]:
            q, k = plain.qk_l2_norm(q, cfg["rms_norm_eps"]), plain.qk_l2_norm(k, cfg["rms_norm_eps"])
        mask = plain.visible_mask(positions, "chunk", cfg["attention_chunk_size"])
    else:
        if cfg["attn_temperature_tuning"]:
            q = q * plain.attn_temperature(positions, cfg["floor_scale"], cfg["attn_scale"])[:, None, None]
        mask = plain.visible_mask(positions, "full")
    o = plain.attention(q, k, v, mask).reshape(T, H_ * hd)
    return o @ W[p + "o_proj.weight"].T


@pytest.mark.parametrize("L", [0, 3])          # a rotating, chunked layer and a NoPE layer
def test_mixer_alone_in_two_portions(rig, L):
    from spite_amd.parts.base import LayerCall
    mixer = rig.eng.model.blocks[L].mixer
    n1, n2 = 37, 30                            # 67 positions: over the chunk borders of both configurations
    x_dev, x_ref = rig.acts(n1 + n2, 5 + L)
    ref = plain_mixer(rig, L, x_ref, torch.arange(n1 + n2))
    slot = rig.eng.admit()
    outs = []
    for a, b in ((0, n1), (n1, n1 + n2)):
        meta = rig.context([(slot, b - a)])
        out = mixer.forward(x_dev[a:b].contiguous(), meta.ctx, meta.layer_cache(rig.eng.cache, LayerCall(L, L, True)))
        outs.append(out.clone())
        rig.commit([(slot, b - a)])
    rig.eng.release(slot)
    rig.close(torch.cat(outs), ref, f"mixer of layer {L}")


def test_feed_forward_alone(rig):
    cfg, W = rig.cfg, rig.w
    _, moe = plain.layer_kinds(cfg)
    T = 19
    for L in (0, 1):
        ffn = rig.eng.model.blocks[L].ffn
        x_dev, x_ref = rig.acts(T, 9 + L)
        meta = rig.context([])
        x32 = x_dev.float()
        outs = ffn.forward(x_dev, x32 if ffn.wants_f32_input else None, meta.ctx)
        f = f"model.layers.{L}.feed_forward."
        if moe[L]:
            ref = plain.moe_ffn(x_ref, W[f + "router.weight"], W[f + "experts.gate_up_proj"], W[f + "experts.down_proj"],
                                W[f + "shared_expert.gate_proj.weight"], W[f + "shared_expert.up_proj.weight"],
                                W[f + "shared_expert.down_proj.weight"])
            assert len(outs) == 2
        else:
            ref = plain.swiglu_mlp(x_ref, W[f + "gate_proj.weight"], W[f + "up_proj.weight"], W[f + "down_proj.weight"])
            assert len(outs) == 1
        rig.close(sum(o.double() for o in outs), ref, f"feed-forward of layer {L}")


def test_moe_reference_vector_through_the_part():
    # crates/spite-models/src/moe.rs:274-292 on the GPU part: 2 experts, x = [1, 2] -> [30, 60]
    from spite_amd.engine.context import Env, Workspace, StepContext, HostBatch
    from spite_amd.parts.feed_forward import MoeTop1Sigmoid
    for dt in (torch.float32, torch.bfloat16):
        env = Env(dt, torch.device(DEV))
        d = 8                                    # the reference's 2, padded with zeros to a width the kernels take
        part = MoeTop1Sigmoid(env, hidden_size=d, intermediate_size=8, n_experts=2)
        router = torch.zeros(2, d); router[1, 1] = 10.0
        gate_up = torch.zeros(2, d, 16); gate_up[1, :2, :2] = 10.0; gate_up[1, 0, 8] = 1.0; gate_up[1, 1, 9] = 1.0
        down = torch.zeros(2, 8, d); down[1, 0, 0] = 1.0; down[1, 1, 1] = 1.0
        z = lambda *s: torch.zeros(*s)
        part.load({k: v.to(DEV).to(torch.float32 if k == "router" else dt) for k, v in {
            "router": router, "experts.gate_up_proj": gate_up, "experts.down_proj": down,
            "shared.gate_proj": z(8, d), "shared.up_proj": z(8, d), "shared.down_proj": z(d, 8)}.items()})
        x = torch.zeros(1, d); x[0, 0], x[0, 1] = 1.0, 2.0
        ctx = StepContext(T=1, n_seqs=1, token_ids=None, positions=None, seq_of_token=None, cu_seqlens=None,
                          seq_slots=None, seq_starts=None, logit_rows=None, n_out=0,
                          host=HostBatch(np.zeros(1), np.zeros(1), np.ones(1), np.array([0, 1])),
                          ws=Workspace(torch.device(DEV), 1 << 20))
        outs = part.forward(x.to(DEV).to(dt), x.to(DEV), ctx)
        y = sum(o.double() for o in outs).cpu()[0]
        assert abs(y[0] - 30.0) < 0.2 and abs(y[1] - 60.0) < 0.4 and y[2:].abs().max() == 0


@pytest.mark.parametrize("T", [9, 32, 33, 48, 64, 65, 150])
def test_experts_with_weights_in_operand_order(T):
    """The experts' part alone at sizes whose weights lie in MFMA operand order (the tiny
    configurations' do not), over the token counts at which it changes its products: few rows
    (one grouped product), 33 to 64 (the shared expert as a product of its own), more (tiles)."""
    from spite_amd.engine.context import Env, Workspace, StepContext, HostBatch
    from spite_amd.parts.feed_forward import MoeTop1Sigmoid
    d, F_, E = 128, 64, 16
    g = torch.Generator().manual_seed(100 + T)
    rnd = lambda *s, std=1.0: torch.randn(*s, generator=g) * std
    w = {"router": rnd(E, d, std=0.5), "experts.gate_up_proj": rnd(E, d, 2 * F_, std=0.1),
         "experts.down_proj": rnd(E, F_, d, std=0.1), "shared.gate_proj": rnd(F_, d, std=0.1),
         "shared.up_proj": rnd(F_, d, std=0.1), "shared.down_proj": rnd(d, F_, std=0.1)}
    w = {k: (v if k == "router" else v.to(torch.bfloat16)) for k, v in w.items()}
    part = MoeTop1Sigmoid(Env(torch.bfloat16, torch.device(DEV)), hidden_size=d, intermediate_size=F_, n_experts=E)
    part.load({k: v.to(DEV) for k, v in w.items()})
    assert part.w_gate_up.tiled and part.w_down.tiled
    x = rnd(T, d).to(torch.bfloat16)
    ctx = StepContext(T=T, n_seqs=1, token_ids=None, positions=None, seq_of_token=None, cu_seqlens=None,
                      seq_slots=None, seq_starts=None, logit_rows=None, n_out=0,
                      host=HostBatch(np.zeros(1), np.zeros(1), np.full(1, T), np.array([0, T])),
                      ws=Workspace(torch.device(DEV), 1 << 24))
    outs = part.forward(x.to(DEV), x.to(DEV).float(), ctx)
    W = {k: v.double() for k, v in w.items()}
    ref = plain.moe_ffn(x.double(), W["router"], W["experts.gate_up_proj"], W["experts.down_proj"],
                        W["shared.gate_proj"], W["shared.up_proj"], W["shared.down_proj"])
    got = sum(o.double() for o in outs).cpu()
    err = (got - ref).abs().max().item()
    assert err <= 1e-2 * ref.abs().max().item(), (T, err, ref.abs().max().item())


@pytest.mark.parametrize("T", [7, 40, 150])
@pytest.mark.parametrize("how", ["shared expert of another width", "shared expert kept in 32-bit"])
def test_experts_with_a_shared_expert_of_its_own(T, how):
    """The experts' part when the shared expert cannot be one more group of the grouped products:
    its intermediate size differs from the routed experts', or the checkpoint kept it in 32-bit
    beside bfloat16 experts.  It then runs as two plain products of its own."""
    from spite_amd.engine.context import Env, Workspace, StepContext, HostBatch
    from spite_amd.parts.feed_forward import MoeTop1Sigmoid
    d, F_, E = 128, 64, 8
    Fs = 96 if how == "shared expert of another width" else F_
    wide = how == "shared expert kept in 32-bit"
    g = torch.Generator().manual_seed(200 + T)
    rnd = lambda *s, std=1.0: torch.randn(*s, generator=g) * std
    w = {"router": rnd(E, d, std=0.5), "experts.gate_up_proj": rnd(E, d, 2 * F_, std=0.1),
         "experts.down_proj": rnd(E, F_, d, std=0.1), "shared.gate_proj": rnd(Fs, d, std=0.1),
         "shared.up_proj": rnd(Fs, d, std=0.1), "shared.down_proj": rnd(d, Fs, std=0.1)}
    w = {k: (v if k == "router" or (wide and k.startswith("shared.")) else v.to(torch.bfloat16)) for k, v in w.items()}
    part = MoeTop1Sigmoid(Env(torch.bfloat16, torch.device(DEV)), hidden_size=d, intermediate_size=F_, n_experts=E,
                          shared_intermediate_size=Fs)
    part.load({k: v.to(DEV) for k, v in w.items()})
    assert not part.fused_shared and part.ws_gate_up is not None
    assert part.ws_gate_up.dtype == (torch.float32 if wide else torch.bfloat16)
    x = rnd(T, d).to(torch.bfloat16)
    ctx = StepContext(T=T, n_seqs=1, token_ids=None, positions=None, seq_of_token=None, cu_seqlens=None,
                      seq_slots=None, seq_starts=None, logit_rows=None, n_out=0,
                      host=HostBatch(np.zeros(1), np.zeros(1), np.full(1, T), np.array([0, T])),
                      ws=Workspace(torch.device(DEV), 1 << 24))
    outs = part.forward(x.to(DEV), x.to(DEV).float(), ctx)
    W = {k: v.double() for k, v in w.items()}
    ref = plain.moe_ffn(x.double(), W["router"], W["experts.gate_up_proj"], W["experts.down_proj"],
                        W["shared.gate_proj"], W["shared.up_proj"], W["shared.down_proj"])
    got = sum(o.double() for o in outs).cpu()
    err = (got - ref).abs().max().item()
    assert err <= 1e-2 * ref.abs().max().item(), (T, how, err, ref.abs().max().item())
    # the shared expert's share alone, so that a shared expert that never ran cannot hide behind the routed one
    alone = plain.swiglu_mlp(x.double(), W["shared.gate_proj"], W["shared.up_proj"], W["shared.down_proj"])
    assert (outs[1].double().cpu() - alone).abs().max().item() <= 1e-2 * alone.abs().max().item()


def test_block_alone(rig):
    from spite_amd.parts.base import LayerCall
    cfg, W = rig.cfg, rig.w
    L, T = 1, 23
    blk = rig.eng.model.blocks[L]
    g = torch.Generator().manual_seed(33)
    h0 = torch.randn(T, rig.d, generator=g)
    slot = rig.eng.admit()
    meta = rig.context([(slot, T)])
    h = h0.to(DEV).clone()
    pending = blk.forward(h, (), meta.ctx, meta.layer_cache(rig.eng.cache, LayerCall(L, L, True)))
    got = h.double().cpu() + sum(p.double().cpu() for p in pending)
    rig.eng.release(slot)
    # plain: h + mixer(norm(h)); then + ffn(norm(.)).  In bfloat16 the part rounds the normed
    # activations before the mixer, the plain side does the same so that only the part's own
    # arithmetic is compared
    rnd = (lambda t: t.to(rig.dt).double())
    p = f"model.layers.{L}."
    eps = cfg["rms_norm_eps"]
    n1 = rnd(plain.rms_norm(h0.double(), W[p + "input_layernorm.weight"], eps))
    h1 = h0.double() + plain_mixer(rig, L, n1, torch.arange(T))
    n2 = rnd(plain.rms_norm(h1, W[p + "post_attention_layernorm.weight"], eps))
    f = p + "feed_forward."
    ref = h1 + plain.moe_ffn(n2, W[f + "router.weight"], W[f + "experts.gate_up_proj"], W[f + "experts.down_proj"],
                             W[f + "shared_expert.gate_proj.weight"], W[f + "shared_expert.up_proj.weight"],
                             W[f + "shared_expert.down_proj.weight"])
    rig.close(got, ref, "block")
