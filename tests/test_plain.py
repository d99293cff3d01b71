"""Pins the plain implementation by what fixes it beside the reference's text: vectors that
the reference's own tests hold, special cases that reduce to a library routine, invariants.
Each is chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong
place, a weight on the wrong side of the expert) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama4 as plain

torch.manual_seed(0)
D = torch.float64


# ------------------------------------------------------------------ norm
def test_rms_norm_is_the_library_routine():
    x, w = torch.randn(5, 48, dtype=D), torch.randn(48, dtype=D)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-12)


def test_rms_norm_invariants():
    x = torch.randn(3, 64, dtype=D)
    y = plain.rms_norm(x, None, 1e-12)
    assert torch.allclose((y * y).mean(-1), torch.ones(3, dtype=D), atol=1e-9)
    assert torch.allclose(plain.rms_norm(7.5 * x, None, 1e-12), y, atol=1e-9)       # scale of x drops out
    # eps is inside the root, beside the mean (not the sum): for x = 0 the result is 0, and
    # for tiny x the result is x/sqrt(eps)
    tiny = torch.full((1, 4), 1e-9, dtype=D)
    assert torch.allclose(plain.rms_norm(tiny, None, 1e-4), tiny / math.sqrt(1e-4 + 1e-18), rtol=1e-9)


# ------------------------------------------------------------------ rotation
def test_rope_hand_vector_pins_pairing_and_sign():
    # hd=4, theta=10000: f = [1, 1/100]; pos 1; x = e0 -> (cos 1, 0, sin 1, 0) under half-split
    inv = plain.rope_inv_freq(4, 10000.0, None)
    assert torch.allclose(inv, torch.tensor([1.0, 0.01], dtype=D))
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]], dtype=D)
    y = plain.apply_rope(x, torch.tensor([1]), inv)
    assert torch.allclose(y[0, 0], torch.tensor([math.cos(1), 0, math.sin(1), 0], dtype=D), atol=1e-12)
    # adjacent pairing moves the partner to index 1
    y2 = plain.apply_rope(x, torch.tensor([1]), inv, "adjacent")
    assert torch.allclose(y2[0, 0], torch.tensor([math.cos(1), math.sin(1), 0, 0], dtype=D), atol=1e-12)
    # second pair turns by the slow frequency: e1 -> (0, cos .03, 0, sin .03) at pos 3
    x = torch.tensor([[[0.0, 1.0, 0.0, 0.0]]], dtype=D)
    y = plain.apply_rope(x, torch.tensor([3]), inv)
    assert torch.allclose(y[0, 0], torch.tensor([0, math.cos(0.03), 0, math.sin(0.03)], dtype=D), atol=1e-12)


def test_rope_invariants():
    inv = plain.rope_inv_freq(16, 500000.0, None)
    q, k = torch.randn(1, 2, 16, dtype=D), torch.randn(1, 2, 16, dtype=D)
    assert torch.equal(plain.apply_rope(q, torch.tensor([0]), inv), q)                     # pos 0: identity
    r = plain.apply_rope(q, torch.tensor([37]), inv)
    assert torch.allclose(r.norm(dim=-1), q.norm(dim=-1), atol=1e-12)                      # a rotation
    def dot(p, j):
        return (plain.apply_rope(q, torch.tensor([p]), inv) * plain.apply_rope(k, torch.tensor([j]), inv)).sum(-1)
    assert torch.allclose(dot(40, 33), dot(107, 100), atol=1e-9)                           # only p - j counts
    assert not torch.allclose(dot(40, 33), dot(40, 30), atol=1e-6)


def test_llama3_scaling():
    base = plain.rope_inv_freq(64, 10000.0, None)
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    assert torch.allclose(plain.rope_inv_freq(64, 10000.0, dict(sc, factor=1.0)), base, atol=1e-15)
    s = plain.rope_inv_freq(64, 10000.0, sc)
    wavelen = 2 * math.pi / base
    high = wavelen < 64 / 4.0
    low = wavelen > 64 / 1.0
    assert high.any() and low.any() and (~high & ~low).any()
    assert torch.equal(s[high], base[high])                   # short waves untouched
    assert torch.allclose(s[low], base[low] / 8.0)            # long waves slowed by the factor
    mid = ~high & ~low
    assert ((s[mid] < base[mid]) & (s[mid] > base[mid] / 8.0)).all()
    with pytest.raises(ValueError):
        plain.rope_inv_freq(64, 10000.0, dict(sc, rope_type="yarn"))


def test_llama3_scaling_is_continuous_and_monotonic_across_the_band():
    # the reference has no frequency scaling, so nothing of its text or tests pins the blend
    # between the two band edges (parity with the reference: unpinned).  What pins it here: the
    # rescaled frequency must join the untouched short waves at one edge (s = 1) and the slowed
    # long waves at the other (s = 0) without a jump, and the ratio to the plain frequency must
    # fall steadily from 1 to 1/factor in between.  A blend with s and 1-s exchanged jumps at both
    # edges and rises in between.  2,048 frequencies make the steps between neighbours small.
    from spite_amd.parts.position import inv_frequencies
    for factor, low, high, orig, theta in ((8.0, 1.0, 4.0, 64, 10000.0), (16.0, 1.0, 4.0, 8192, 500000.0)):
        sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
                  original_max_position_embeddings=orig)
        base = plain.rope_inv_freq(4096, theta, None)
        ratio = plain.rope_inv_freq(4096, theta, sc) / base
        wavelen = 2 * math.pi / base
        band = (wavelen >= orig / high) & (wavelen <= orig / low)
        assert 20 < int(band.sum()) < 2000
        assert float(ratio.max()) == 1.0 and abs(float(ratio.min()) - 1.0 / factor) < 1e-12
        steps = ratio[1:] - ratio[:-1]                       # frequencies fall with the index
        assert (steps <= 1e-15).all(), "the ratio must never rise from short waves to long ones"
        assert float(steps.abs().max()) < 3.0 * (1.0 - 1.0 / factor) / int(band.sum()), "a jump at a band edge"
        # the engine's table is the same function
        mine = torch.tensor(inv_frequencies(4096, theta, sc), dtype=torch.float64)
        assert torch.allclose(mine, plain.rope_inv_freq(4096, theta, sc), rtol=1e-13, atol=0)
        mine = torch.tensor(inv_frequencies(128, theta, sc), dtype=torch.float64)
        assert torch.allclose(mine, plain.rope_inv_freq(128, theta, sc), rtol=1e-13, atol=0)


def test_qk_norm_commutes_with_rotation():
    inv = plain.rope_inv_freq(8, 100.0, None)
    x = torch.randn(4, 3, 8, dtype=D)
    pos = torch.tensor([0, 5, 9, 31])
    a = plain.qk_l2_norm(plain.apply_rope(x, pos, inv), 1e-6)
    b = plain.apply_rope(plain.qk_l2_norm(x, 1e-6), pos, inv)
    assert torch.allclose(a, b, atol=1e-12)
    assert torch.allclose((a * a).mean(-1), torch.ones(4, 3, dtype=D), atol=1e-4)


def test_temperature_steps_at_multiples_of_floor_scale():
    pos = torch.arange(0, 50)
    s = plain.attn_temperature(pos, 16, 0.1)
    assert torch.all(s[:15] == 1.0)                            # pos+1 < 16
    assert s[15] == pytest.approx(math.log(2) * 0.1 + 1)       # pos+1 == 16
    assert s[30] == s[15] and s[31] == pytest.approx(math.log(3) * 0.1 + 1)
    # the reference's constants (llama4.rs:179)
    assert float(plain.attn_temperature(torch.tensor([8191]), 8192, 0.1)[0]) == pytest.approx(math.log(2) * 0.1 + 1)
    assert float(plain.attn_temperature(torch.tensor([8190]), 8192, 0.1)[0]) == 1.0


# ------------------------------------------------------------------ attention
def test_attention_reference_vector():
    # crates/spite-compute/src/flash_attn.rs:164-174: one token, Q = K = V = 1 -> 1
    o = plain.attention(torch.ones(1, 2, 4, dtype=D), torch.ones(1, 2, 4, dtype=D), torch.ones(1, 2, 4, dtype=D),
                        plain.visible_mask(torch.tensor([0]), "full"))
    assert torch.allclose(o, torch.ones(1, 2, 4, dtype=D), atol=1e-12)


@pytest.mark.parametrize("H,G", [(4, 4), (6, 2), (3, 1)])
def test_attention_is_the_library_routine_without_rotation(H, G):
    T, hd = 9, 8
    q, k, v = torch.randn(T, H, hd, dtype=D), torch.randn(T, G, hd, dtype=D), torch.randn(T, G, hd, dtype=D)
    mine = plain.attention(q, k, v, plain.visible_mask(torch.arange(T), "full"))
    kk = k.repeat_interleave(H // G, dim=1).transpose(0, 1)
    vv = v.repeat_interleave(H // G, dim=1).transpose(0, 1)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, is_causal=True).transpose(0, 1)
    assert torch.allclose(mine, lib, atol=1e-12)


def test_visibility_rules():
    pos = torch.arange(10)
    full, chunk, win = (plain.visible_mask(pos, "full"), plain.visible_mask(pos, "chunk", 4),
                        plain.visible_mask(pos, "window", 4))
    assert torch.equal(full, torch.tril(torch.ones(10, 10, dtype=torch.bool)))
    assert torch.equal(plain.visible_mask(pos, "chunk", 16), full)         # chunk >= length: causal
    assert chunk[5].tolist() == [False] * 4 + [True, True] + [False] * 4   # keys 4,5
    assert chunk[4].tolist() == [False] * 4 + [True] + [False] * 5         # first of a chunk: itself only
    assert win[5].tolist() == [False, False, True, True, True, True] + [False] * 4  # the last 4 rows
    assert not torch.equal(chunk, win)
    # shifted positions: the rule uses absolute positions
    assert plain.visible_mask(torch.arange(6, 9), "chunk", 4).tolist() == [[True, False, False], [True, True, False],
                                                                              [False, False, True]]


def test_first_token_of_a_chunk_returns_its_own_value():
    T, H, hd = 12, 2, 4
    q, k, v = torch.randn(T, H, hd, dtype=D), torch.randn(T, H, hd, dtype=D), torch.randn(T, H, hd, dtype=D)
    o = plain.attention(q, k, v, plain.visible_mask(torch.arange(T), "chunk", 4))
    for t in (0, 4, 8):
        assert torch.allclose(o[t], v[t], atol=1e-12)


# ------------------------------------------------------------------ feed-forward
def test_dense_mlp_is_silu_times_up_then_down():
    x = torch.randn(5, 12, dtype=D)
    wg, wu, wd = torch.randn(20, 12, dtype=D), torch.randn(20, 12, dtype=D), torch.randn(12, 20, dtype=D)
    lib = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain.swiglu_mlp(x, wg, wu, wd), lib, atol=1e-12)


def _no_shared(d, F_):
    z = torch.zeros(F_, d, dtype=D)
    return z, z, torch.zeros(d, F_, dtype=D)


def test_moe_reference_vector():
    # crates/spite-models/src/moe.rs:274-292: 2 experts, router rows [0,0] and [0,10], x = [1,2]
    # -> expert 1, weight sigmoid(20) ~ 1, gate = [30,30], up = [1,2], out ~ [30,60]
    router = torch.tensor([[0.0, 0.0], [0.0, 10.0]], dtype=D)
    ident = torch.eye(2, dtype=D)
    gate_up = torch.zeros(2, 2, 4, dtype=D)          # [E, d, 2F]
    gate_up[1, :, :2] = 10.0                         # gate rows all 10 -> x @ M = 10*(x0+x1)
    gate_up[1, :, 2:] = ident                        # up = identity
    down = torch.zeros(2, 2, 2, dtype=D)
    down[1] = ident
    x = torch.tensor([[1.0, 2.0]], dtype=D)
    idx, w, logits = plain.router_top1(x, router)
    assert idx.tolist() == [1] and logits.tolist() == [[0.0, 20.0]] and float(w[0]) == pytest.approx(1.0, abs=1e-8)
    y = plain.moe_ffn(x, router, gate_up, down, *_no_shared(2, 2))
    assert torch.allclose(y, torch.tensor([[30.0, 60.0]], dtype=D), atol=1e-6)


def test_router_ties_go_to_the_lowest_index():
    router = torch.tensor([[1.0, 0.0], [2.0, 0.0], [2.0, 0.0], [0.5, 0.0]], dtype=D)
    idx, w, _ = plain.router_top1(torch.tensor([[1.0, 3.0]], dtype=D), router)
    assert idx.tolist() == [1] and float(w[0]) == pytest.approx(1 / (1 + math.exp(-2.0)))
    # the library's top-1 picks the same value
    assert float(torch.topk(torch.tensor([1.0, 2.0, 2.0, 0.5]), 1).values[0]) == 2.0


def test_moe_weight_scales_the_input_not_the_output():
    d, F_, E = 6, 10, 1
    x = torch.randn(4, d, dtype=D)
    router = torch.randn(E, d, dtype=D)
    gate_up, down = torch.randn(E, d, 2 * F_, dtype=D), torch.randn(E, F_, d, dtype=D)
    sg, su, sd = torch.randn(F_, d, dtype=D), torch.randn(F_, d, dtype=D), torch.randn(d, F_, dtype=D)
    y = plain.moe_ffn(x, router, gate_up, down, sg, su, sd)
    w = torch.sigmoid(x @ router.T)                                        # [T,1]
    def expert(z):
        gu = z @ gate_up[0]
        return (F.silu(gu[:, :F_]) * gu[:, F_:]) @ down[0]
    shared = F.linear(F.silu(F.linear(x, sg)) * F.linear(x, su), sd)
    assert torch.allclose(y, expert(x * w) + shared, atol=1e-10)           # one expert: expert(sigma(r) x) + shared(x)
    assert not torch.allclose(y, w * expert(x) + shared, atol=1e-3)        # not the post-weighted form
    assert not torch.allclose(y, expert(x * w) + F.linear(F.silu(F.linear(x * w, sg)) * F.linear(x * w, su), sd),
                              atol=1e-3)                                   # the shared expert sees the unscaled x


def test_identical_experts_with_a_sure_router_are_a_plain_mlp():
    d, F_, E = 6, 8, 3
    x = torch.randn(5, d, dtype=D)
    one_gu, one_dn = torch.randn(d, 2 * F_, dtype=D), torch.randn(F_, d, dtype=D)
    gate_up, down = one_gu.expand(E, -1, -1).contiguous(), one_dn.expand(E, -1, -1).contiguous()
    router = torch.zeros(E, d, dtype=D)
    router[2] = 1e3 * x.mean(0).sign()                                     # a huge logit for one expert
    x = x.abs() * x.mean(0).sign()                                         # so that it is huge for every row
    y = plain.moe_ffn(x, router, gate_up, down, *_no_shared(d, F_))
    mlp = plain.swiglu_mlp(x, one_gu[:, :F_].T, one_gu[:, F_:].T, one_dn.T)
    assert torch.allclose(y, mlp, atol=1e-9)


# ------------------------------------------------------------------ whole model
def _tiny_reference_model():
    """The constant-filled two-layer model of crates/spite-models/src/llama/llama4.rs:290-359
    (layer 0 dense, layer 1 with 4 experts top-1), under this repository's tensor names."""
    d, hd, nh, ff, ffe, v, ne = 8, 4, 2, 16, 8, 8, 4
    cfg = dict(num_hidden_layers=2, hidden_size=d, num_attention_heads=nh, num_key_value_heads=nh, head_dim=hd,
               intermediate_size=ffe, intermediate_size_mlp=ff, vocab_size=v, rope_theta=10000.0, rms_norm_eps=1e-5,
               num_local_experts=ne, num_experts_per_tok=1, interleave_moe_layer_step=2, no_rope_layers=[1, 1],
               attention_chunk_size=None, use_qk_norm=True, attn_temperature_tuning=False)
    full = lambda r, c, x: torch.full((r, c), x, dtype=D)
    W = {"model.embed_tokens.weight": full(v, d, 0.1), "model.norm.weight": torch.ones(d, dtype=D),
         "lm_head.weight": full(v, d, 0.1)}
    for L in range(2):
        p = f"model.layers.{L}."
        W[p + "input_layernorm.weight"] = torch.ones(d, dtype=D)
        W[p + "post_attention_layernorm.weight"] = torch.ones(d, dtype=D)
        for n in ("q_proj", "k_proj", "v_proj"):
            W[p + f"self_attn.{n}.weight"] = full(nh * hd, d, 0.05)
        W[p + "self_attn.o_proj.weight"] = full(d, nh * hd, 0.05)
        f = p + "feed_forward."
        if L == 1:
            W[f + "router.weight"] = full(ne, d, 0.5)
            W[f + "experts.gate_up_proj"] = torch.full((ne, d, 2 * ffe), 0.05, dtype=D)
            W[f + "experts.down_proj"] = torch.full((ne, ffe, d), 0.05, dtype=D)
            W[f + "shared_expert.gate_proj.weight"] = full(ffe, d, 0.05)
            W[f + "shared_expert.up_proj.weight"] = full(ffe, d, 0.05)
            W[f + "shared_expert.down_proj.weight"] = full(d, ffe, 0.05)
        else:
            W[f + "gate_proj.weight"] = full(ff, d, 0.05)
            W[f + "up_proj.weight"] = full(ff, d, 0.05)
            W[f + "down_proj.weight"] = full(d, ff, 0.05)
    return cfg, W


def test_reference_tiny_model_whole_equals_incremental():
    # llama4.rs:361-390: forward([1,2]) against forward([1]) then forward([2]) at pos 1.  The
    # plain implementation has no cache; the same statement is: a prefix's logits do not
    # change when tokens follow it, and a start position moves the rotation only.
    cfg, W = _tiny_reference_model()
    full = plain.forward(cfg, W, [1, 2])
    assert torch.isfinite(full).all()
    assert torch.allclose(plain.forward(cfg, W, [1]), full[:1], atol=1e-12)
    # with constant fills every token embeds alike, the router ties, and expert 0 is taken
    n = plain.rms_norm(W["model.embed_tokens.weight"][[1]], None, 1e-5)
    idx, _, _ = plain.router_top1(n, W["model.layers.1.feed_forward.router.weight"])
    assert idx.tolist() == [0]


def test_untied_head_does_not_touch_hidden_states_and_tied_head_is_the_embedding():
    cfg, W = _tiny_reference_model()
    a = plain.forward(cfg, W, [1, 2, 3])
    W2 = dict(W)
    W2["lm_head.weight"] = 2.0 * W["lm_head.weight"]
    assert torch.allclose(plain.forward(cfg, W2, [1, 2, 3]), 2.0 * a, atol=1e-12)
    W3 = {k: v for k, v in W.items() if k != "lm_head.weight"}
    assert torch.allclose(plain.forward(dict(cfg, tie_word_embeddings=True), W3, [1, 2, 3]), a, atol=1e-12)


def test_positions_shift_only_moves_chunks_and_temperature():
    # No chunking, no temperature: a shift of every position leaves the logits alone,
    # because rotation enters through differences of positions only.
    from helpers import TINY_B, planted_tensors
    cfg = dict(TINY_B, attention_chunk_size=None, num_hidden_layers=4)
    W = {k: v.to(D) for k, v in planted_tensors(cfg, 5).items()}
    toks = list(range(3, 23))
    a = plain.forward(cfg, W, toks, start_pos=0)
    b = plain.forward(cfg, W, toks, start_pos=11)
    assert torch.allclose(a, b, atol=1e-9)
    # with chunks the shift moves the chunk borders and the logits change
    c = plain.forward(dict(cfg, attention_chunk_size=16), W, toks, start_pos=11)
    assert not torch.allclose(a, c, atol=1e-4)


def test_wanted_rows_alone_and_blocks_of_queries_equal_the_whole():
    from helpers import TINY_A, TINY_B, planted_tensors
    for cfg, kind in ((TINY_A, None), (TINY_B, "window"), (dict(TINY_B, attention_local_kind="window"), None)):
        W = {k: v.to(D) for k, v in planted_tensors(cfg, 3).items()}
        toks = [(7 * i + 3) % cfg["vocab_size"] for i in range(75)]
        whole = plain.forward(cfg, W, toks, start_pos=5, visibility=kind)
        rows = [5, 6, 20, 36, 37, 52, 79]
        some = plain.forward(cfg, W, toks, start_pos=5, visibility=kind, rows=rows)
        assert torch.allclose(some, whole[[r - 5 for r in rows]], atol=1e-12)
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(90, n, 8, generator=g, dtype=D) for n in (4, 2, 2))
    pos = torch.arange(30, 120)
    for kind, size in (("full", 0), ("chunk", 16), ("window", 11)):
        whole = plain.attention(q, k, v, plain.visible_mask(pos, kind, size))
        assert torch.allclose(plain.attention_rows(q, k, v, pos, kind, size, key_start=30, block=7), whole, atol=1e-12)
        pick = torch.tensor([0, 3, 50, 89])
        assert torch.allclose(plain.attention_rows(q[pick], k, v, pos[pick], kind, size, key_start=30, block=3),
                              whole[pick], atol=1e-12)


def test_layer_kinds():
    rope, moe = plain.layer_kinds(dict(num_hidden_layers=8, interleave_moe_layer_step=2))
    assert rope == [True, True, True, False] * 2 and moe == [False, True] * 4
    rope, moe = plain.layer_kinds(dict(num_hidden_layers=4, no_rope_layers=[1, 1, 1, 0], interleave_moe_layer_step=1))
    assert rope == [True, True, True, False] and moe == [True] * 4


# ------------------------------------------------------------------ sampling
def test_sampling_reference_vectors():
    # crates/spite-sampling/src/lib.rs:354-369
    l = plain.apply_top_k(torch.tensor([1.0, 5.0, 3.0, 2.0, 4.0]), 2)
    assert torch.isfinite(l).tolist() == [False, True, False, False, True]
    l = plain.apply_top_p(torch.tensor([2.0, 1.0, 0.0, -2.0]), 0.8)
    assert torch.isfinite(l).tolist() == [True, True, False, False]
    # crates/spite-executor/src/lib.rs:814-828: greedy is the raw arg-max; a penalty can change it
    assert plain.sample(torch.tensor([0.0, 2.0, 1.95]), [1], 0x12345678, 0.0)[0] == 1
    assert plain.sample(torch.tensor([0.0, 2.0, 1.95]), [1], 0x12345678, 0.0, repetition_penalty=1.1)[0] == 2
    # :391-410: each distinct id once; the window
    l = plain.apply_repetition_penalty(torch.tensor([0.0, 3.0, 2.0]), [1, 1, 1], 1.1)
    assert float(l[1]) == pytest.approx(3.0 / 1.1) and float(l[2]) == 2.0
    assert float(plain.apply_repetition_penalty(torch.tensor([0.0, 3.0]), [1, 7, 7], 1.1, 2)[1]) == 3.0
    assert float(plain.apply_min_p(torch.tensor([0.0, -1.0, -5.0]), 0.1)[2]) == float("-inf")
    assert float(plain.apply_min_p(torch.tensor([0.0, -1.0, -5.0]), 0.1)[1]) == -1.0


def test_greedy_takes_the_first_of_equal_maxima():
    assert plain.greedy(torch.tensor([1.0, 3.0, 3.0, 2.0])) == 1
    assert plain.greedy(torch.tensor([float("-inf"), float("-inf")])) == 0


def test_lcg_and_multinomial():
    # the generator of crates/spite-sampling/src/lib.rs:343-348, recomputed with wrapping uint64
    s = np.uint64(42)
    with np.errstate(over="ignore"):
        s = s * np.uint64(6364136223846793005) + np.uint64(1442695040888963407)
    state, u = plain.lcg_next(42)
    assert state == int(s) and u == pytest.approx(float(int(s) >> 33) / 2147483648.0) and 0.0 <= u < 1.0
    # :371-389: the same seed draws the same tokens; the largest logit dominates
    logits = torch.tensor([1.0, 2.0, 3.0])
    def draws(seed, n):
        out, st = [], seed
        for _ in range(n):
            t, st = plain.multinomial(logits, st)
            out.append(t)
        return out
    assert draws(42, 10) == draws(42, 10)
    assert sum(t == 2 for t in draws(1, 200)) > 100
    # temperature -> 0 approaches greedy
    assert all(plain.sample(logits, [], 7 + i, 1e-3)[0] == 2 for i in range(5))
