"""Llama 4 text model as a list of parts.

Layer L rotates and reads the keys of its chunk when ``no_rope_layers[L]`` is 1; otherwise
it has no position encoding, reads every key and scales its queries with the position
(crates/spite-models/src/llama/llama4.rs:155-183).  Layer L has experts when it is listed
in ``moe_layers`` ((L+1) % interleave_moe_layer_step == 0, llama4.rs:44-47), else a dense
gated MLP of width ``intermediate_size_mlp``.
"""
from __future__ import annotations

from .llama4 import Llama4Config
from .registry import register_architecture
from ..parts.base import PartSpec, BlockSpec, LayerCall, ModelSpec


def build_spec(cfg: Llama4Config, ignore_prefixes=()) -> ModelSpec:
    d, H, G, hd = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    scaling = None
    if cfg.rope_scaling is not None:
        rs = cfg.rope_scaling
        scaling = {"rope_type": rs.rope_type, "factor": rs.factor, "low_freq_factor": rs.low_freq_factor,
                   "high_freq_factor": rs.high_freq_factor,
                   "original_max_position_embeddings": rs.original_max_position_embeddings}
    moe = set(cfg.moe_layers)
    blocks = []
    for L in range(cfg.num_hidden_layers):
        p = f"model.layers.{L}."
        rotates = bool(cfg.no_rope_layers[L])
        if rotates:
            position = PartSpec("rotary", {"head_dim": hd, "theta": cfg.rope_theta, "scaling": scaling,
                                           "pairing": cfg.rope_pairing})
            chunked = cfg.attention_chunk_size is not None
            attn_args = dict(visibility=cfg.attention_local_kind if chunked else "full", span=cfg.attention_chunk_size or 0,
                             qk_norm=cfg.use_qk_norm, qk_norm_eps=cfg.rms_norm_eps, temperature=None)
        else:
            position = PartSpec("none")
            temp = (cfg.floor_scale, cfg.attn_scale) if cfg.attn_temperature_tuning else None
            attn_args = dict(visibility="full", span=0, qk_norm=False, qk_norm_eps=cfg.rms_norm_eps,
                             temperature=temp)
        mixer = PartSpec("attention", dict(hidden_size=d, n_heads=H, n_kv_heads=G, head_dim=hd,
                                           position=position, **attn_args),
                         {k: f"{p}self_attn.{k}.weight" for k in ("q_proj", "k_proj", "v_proj", "o_proj")})
        if L in moe:
            f = p + "feed_forward."
            ffn = PartSpec("moe_top1_sigmoid",
                           dict(hidden_size=d, intermediate_size=cfg.intermediate_size,
                                n_experts=cfg.num_local_experts),
                           {"router": f + "router.weight",
                            "experts.gate_up_proj": f + "experts.gate_up_proj",
                            "experts.down_proj": f + "experts.down_proj",
                            "shared.gate_proj": f + "shared_expert.gate_proj.weight",
                            "shared.up_proj": f + "shared_expert.up_proj.weight",
                            "shared.down_proj": f + "shared_expert.down_proj.weight"})
        else:
            f = p + "feed_forward."
            ffn = PartSpec("dense_glu", dict(hidden_size=d, intermediate_size=cfg.intermediate_size_mlp),
                           {k: f"{f}{k}.weight" for k in ("gate_proj", "up_proj", "down_proj")})
        norm = lambda name: PartSpec("rms", {"width": d, "eps": cfg.rms_norm_eps}, {"weight": p + name + ".weight"})
        blocks.append(BlockSpec("prenorm", norm("input_layernorm"), mixer, norm("post_attention_layernorm"), ffn))
    return ModelSpec(
        architecture=cfg.architecture, vocab_size=cfg.vocab_size, hidden_size=d, blocks=blocks,
        order=[LayerCall(block=i, cache=i, write=True) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rms", {"width": d, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
        embed_name="model.embed_tokens.weight",
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        eos_token_ids=cfg.eos_token_ids, max_position=cfg.max_position_embeddings,
        ignore_prefixes=tuple(ignore_prefixes))


def build_text_spec_of_multimodal(cfg: Llama4Config) -> ModelSpec:
    """The text model of a checkpoint that also holds a vision tower: its keys lie under
    ``text_config``, its tensors under ``language_model.``; the other towers' tensors belong to
    no part of this model and are passed over."""
    return build_spec(cfg, ignore_prefixes=("vision_model.", "multi_modal_projector."))


register_architecture("Llama4ForCausalLM", Llama4Config.from_dict, build_spec)
register_architecture("Llama4ForConditionalGeneration", Llama4Config.from_dict, build_text_spec_of_multimodal)
