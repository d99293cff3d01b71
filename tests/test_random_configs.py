"""Random tiny configurations of the architecture, drawn from a seed: head sizes in steps of
16, one to four kv heads with one to eight query heads each, widths and vocabularies that are
no power of two (some no multiple of eight), one to seventeen experts, experts in every, every
second or every third layer, chunks that are no multiple of the page, tied and untied output
matrices.  Each runs whole, in portions of changing size and mixed on a small pool, in 32-bit,
against the plain implementation; the sizes pick the kernels, so this is where a kernel that
mishandles a size it claims to take would show."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def random_config(seed: int):
    r = np.random.RandomState(1000 + seed)
    pick = lambda xs: r.choice(xs).item()
    G, L = pick([1, 2, 3, 4]), pick([1, 2, 3, 4, 5, 6])
    interval = pick([2, 3, 4])
    scaling = None
    if r.rand() < 0.5:
        scaling = dict(rope_type="llama3", factor=pick([2.0, 8.0, 16.0]), low_freq_factor=1.0,
                       high_freq_factor=pick([2.0, 4.0]), original_max_position_embeddings=pick([32, 64, 128]))
    cfg = dict(architectures=["Llama4ForCausalLM"], num_hidden_layers=L,
               hidden_size=pick([40, 64, 72, 96, 100, 128, 136, 192, 256]),
               num_attention_heads=G * pick([1, 2, 3, 4, 5, 7, 8]), num_key_value_heads=G,
               head_dim=pick([16, 32, 48, 64, 80, 96, 112, 128]), rms_norm_eps=pick([1e-5, 1e-6, 1e-4]),
               num_local_experts=pick([1, 2, 3, 4, 5, 8, 16, 17]), num_experts_per_tok=1,
               intermediate_size=pick([16, 24, 40, 64, 72, 128]), intermediate_size_mlp=pick([32, 48, 80, 128, 200]),
               interleave_moe_layer_step=pick([1, 1, 2, 3]), vocab_size=pick([50, 97, 128, 256, 301, 1000, 2049]),
               rope_theta=pick([10000.0, 500000.0, 100.0]), rope_scaling=scaling,
               attention_chunk_size=pick([8, 16, 24, 32, 64, 100]),
               no_rope_layers=[int((i + 1) % interval != 0) for i in range(L)],
               use_qk_norm=bool(r.rand() < 0.5), attn_temperature_tuning=bool(r.rand() < 0.5),
               floor_scale=pick([4, 16, 50]), attn_scale=pick([0.1, 0.3]),
               tie_word_embeddings=bool(r.rand() < 0.25), torch_dtype="float32")
    return cfg, pick([8, 16, 32, 64])


@pytest.mark.parametrize("seed", range(10))
def test_a_random_configuration_in_32_bit(seed, tmp_path):
    from spite_amd.engine.engine import Engine
    cfg, page = random_config(seed)
    weights = H.make_model(str(tmp_path), cfg, seed=seed, dtype="float32")
    lens = [int(n) for n in np.random.RandomState(seed).choice([1, 2, 17, 33, 70, 131, 200], size=4)]
    reqs = {f"r{i}": H.random_tokens(cfg["vocab_size"], n, seed * 10 + i) for i, n in enumerate(lens)}
    ref = H.plain_logits(cfg, weights, reqs)
    scale = max(1.0, max(float(np.abs(v).max()) for v in ref.values()))
    up = lambda n: -(-n // page) * page
    one, three = up(max(lens)), sum(sorted((up(n) for n in lens), reverse=True)[:3])
    for label, steps, pool in (("whole", H.schedule_whole(reqs), one), ("portions", H.schedule_portions(reqs), one),
                               ("mixed", H.schedule_mixed(reqs, seed=seed, max_live=3), three)):
        eng = Engine(str(tmp_path), dtype="float32", page_size=page, cache_tokens=pool, max_requests=4)
        rows = H.collect(steps, H.run_trace_inprocess(eng, steps), cfg["vocab_size"])
        assert all(eng.cache.free_pages(g) == eng.cache.total_pages(g) for g in range(eng.cache.n_groups()))
        d, where = H.max_diff(rows, ref)
        assert d <= 3e-5 * scale, f"{label}: {d} at {where} (logits up to {scale}); {cfg}"
        del eng


def random_config_bf16(seed: int):
    """Sizes that the bfloat16 kernels of serving take: head sizes 64 and 128 with pages of 32 or
    64 (MFMA attention; one seed in four draws another head size and runs the generic kernel),
    widths that are multiples of 64 (weights in operand order), of 8 only (row-major MFMA
    products) or of neither (the generic product)."""
    r = np.random.RandomState(2000 + seed)
    pick = lambda xs: r.choice(xs).item()
    cfg, _ = random_config(seed)
    G = pick([1, 2, 3])
    cfg.update(hidden_size=pick([64, 128, 192, 256, 72, 136, 100]), num_key_value_heads=G,
               num_attention_heads=G * pick([1, 2, 4, 5, 8]), head_dim=pick([64, 128, 64, 128, 64, 128, 32, 96]),
               intermediate_size=pick([64, 128, 192, 72, 40]), intermediate_size_mlp=pick([64, 128, 80, 200]),
               vocab_size=pick([128, 301, 1000, 2049]), attention_chunk_size=pick([32, 64, 96, 128, 100]),
               tie_word_embeddings=bool(seed % 3 == 0), torch_dtype="bfloat16")
    return cfg, pick([32, 64])


@pytest.mark.parametrize("seed", range(8))
def test_a_random_configuration_in_bfloat16(seed, tmp_path):
    from spite_amd.engine.engine import Engine
    cfg, page = random_config_bf16(seed)
    weights = H.make_model(str(tmp_path), cfg, seed=seed, dtype="bfloat16")
    lens = [int(n) for n in np.random.RandomState(seed).choice([1, 2, 17, 33, 70, 131, 200, 300], size=4)]
    reqs = {f"r{i}": H.random_tokens(cfg["vocab_size"], n, seed * 10 + i) for i, n in enumerate(lens)}
    up = lambda n: -(-n // page) * page
    one, three = up(max(lens)), sum(sorted((up(n) for n in lens), reverse=True)[:3])
    n_choices = sum(lens) * len(H.moe_layers(cfg))
    for label, steps, pool in (("whole", H.schedule_whole(reqs), one), ("portions", H.schedule_portions(reqs), one),
                               ("mixed", H.schedule_mixed(reqs, seed=seed, max_live=3), three)):
        eng = Engine(str(tmp_path), dtype="bfloat16", page_size=page, cache_tokens=pool, max_requests=4)
        routing = {}
        rows = H.collect(steps, H.run_trace_inprocess(eng, steps, routing), cfg["vocab_size"])
        assert all(eng.cache.free_pages(g) == eng.cache.total_pages(g) for g in range(eng.cache.n_groups()))
        # the plain implementation follows the engine's expert where its own best two are tied at
        # bfloat16's precision (see test_replay.py)
        taken = []
        ref = H.plain_logits(cfg, weights, reqs, H.routing_hints(cfg, steps, routing), 0.04, taken)
        scale = max(float(np.abs(v).max()) for v in ref.values())
        d, where = H.max_diff(rows, ref)
        print(f"[bf16 config {seed}] {label}: {d / scale:.2%} of the scale at {where}; {len(taken)} of {n_choices} near ties; "
              f"d={cfg['hidden_size']} hd={cfg['head_dim']} H={cfg['num_attention_heads']}/{cfg['num_key_value_heads']} "
              f"F={cfg['intermediate_size']} V={cfg['vocab_size']} tied={cfg['tie_word_embeddings']} page={page}")
        assert d <= 0.04 * scale, f"{label}: {d} at {where} (logits up to {scale}); {cfg}"
        assert len(taken) <= max(3, 0.03 * n_choices)
        del eng
