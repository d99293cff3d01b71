"""Configuration: reading config.json keys into the typed configuration, one error that
lists every problem, the architecture registry, the layer list that the spec derives."""
import json

import pytest

from helpers import TINY_A, TINY_B
from spite_amd.config import (Llama4Config, ConfigError, read_config, registered_architectures,
                              UnknownArchitecture, architecture)


def test_reads_every_key_of_both_tiny_configurations():
    a, b = Llama4Config.from_dict(TINY_A), Llama4Config.from_dict(TINY_B)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (4, 64, 4, 2, 16)
    assert (b.num_hidden_layers, b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim) == (8, 96, 6, 3, 24)
    assert a.rms_norm_eps == 1e-5 and b.rms_norm_eps == 1e-6
    assert a.no_rope_layers == (1, 1, 1, 0) and b.no_rope_layers == (1, 1, 1, 0, 1, 1, 1, 0)   # every 4th is NoPE
    assert a.moe_layers == (0, 1, 2, 3) and b.moe_layers == (1, 3, 5, 7)
    assert a.rope_scaling is None and b.rope_scaling.factor == 8.0 and b.rope_scaling.original_max_position_embeddings == 64
    assert (a.attention_chunk_size, b.attention_chunk_size) == (32, 16)
    assert a.use_qk_norm and not b.use_qk_norm and a.attn_temperature_tuning and not b.attn_temperature_tuning
    assert (a.floor_scale, a.attn_scale) == (16, 0.1)
    assert b.head_dim != b.hidden_size // b.num_attention_heads       # the head size is a key of its own


def test_defaults_follow_the_reference():
    cfg = Llama4Config.from_dict(dict(architectures=["Llama4ForCausalLM"], num_hidden_layers=2, hidden_size=32,
                                      num_attention_heads=4, vocab_size=10, intermediate_size_mlp=8,
                                      num_local_experts=0))
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 10000.0        # crates/spite-loader/src/config.rs:147-154
    assert cfg.head_dim == 8 and cfg.num_key_value_heads == 4
    assert (cfg.floor_scale, cfg.attn_scale) == (8192, 0.1)              # crates/spite-models/src/llama/llama4.rs:179
    assert cfg.moe_layers == () and not cfg.tie_word_embeddings


def test_text_config_nesting_and_unknown_keys():
    cfg = Llama4Config.from_dict({"architectures": ["Llama4ForCausalLM"], "text_config": dict(TINY_A, some_new_key=3)})
    assert cfg.hidden_size == 64


def test_one_error_lists_every_problem():
    bad = dict(TINY_A, num_attention_heads=5, head_dim=15, no_rope_layers=[1, 0], num_experts_per_tok=2)
    del bad["vocab_size"]
    with pytest.raises(ConfigError) as e:
        Llama4Config.from_dict(bad)
    msg = str(e.value)
    for piece in ("vocab_size", "not a multiple", "head_dim 15", "no_rope_layers has 2", "top-1"):
        assert piece in msg, msg


@pytest.mark.parametrize("key,val", [("rms_norm_eps", 0.0), ("attention_chunk_size", -4), ("rope_pairing", "odd"),
                                     ("floor_scale", 0), ("torch_dtype", "int8"), ("hidden_size", "wide")])
def test_bad_values_are_refused(key, val):
    with pytest.raises(ConfigError):
        Llama4Config.from_dict(dict(TINY_A, **{key: val}))


def test_rope_scaling_of_unknown_type_is_refused():
    with pytest.raises(ConfigError, match="yarn"):
        Llama4Config.from_dict(dict(TINY_B, rope_scaling=dict(rope_type="yarn", factor=2.0)))


def test_registry(tmp_path):
    assert "Llama4ForCausalLM" in registered_architectures()
    with pytest.raises(UnknownArchitecture, match="Llama4ForCausalLM"):
        architecture("GPT2LMHeadModel")
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    arch, cfg = read_config(str(tmp_path))
    assert arch.name == "Llama4ForCausalLM" and cfg.vocab_size == 384
    with pytest.raises(UnknownArchitecture):
        read_config(dict(TINY_A, architectures=["NoSuchModel"]))


def test_spec_chooses_parts_layer_by_layer():
    arch, cfg = read_config(TINY_B)
    spec = arch.build_spec(cfg)
    assert len(spec.blocks) == 8 and [c.block for c in spec.order] == list(range(8))
    kinds = [(b.mixer.args["position"].kind, b.mixer.args["visibility"], b.ffn.kind) for b in spec.blocks]
    assert kinds[0] == ("rotary", "chunk", "dense_glu") and kinds[1] == ("rotary", "chunk", "moe_top1_sigmoid")
    assert kinds[3] == ("none", "full", "moe_top1_sigmoid") and kinds[6] == ("rotary", "chunk", "dense_glu")
    assert spec.blocks[0].mixer.args["span"] == 16 and spec.blocks[3].mixer.args["temperature"] is None
    a = read_config(TINY_A)[0].build_spec(Llama4Config.from_dict(TINY_A))
    assert a.blocks[3].mixer.args["temperature"] == (16, 0.1) and a.blocks[0].mixer.args["qk_norm"]
    assert not a.blocks[3].mixer.args["qk_norm"]                         # qk-norm on rotating layers only


def test_round_trip_through_to_dict():
    cfg = Llama4Config.from_dict(TINY_B)
    assert Llama4Config.from_dict(cfg.to_dict()) == cfg
