"""Typed Llama 4 text configuration, read from the keys of its ``config.json``.

Key map from the reference's GGUF metadata (crates/spite-loader/src/config.rs:228-343):
``block_count`` -> ``num_hidden_layers``; ``embedding_length`` -> ``hidden_size``;
``attention.head_count`` -> ``num_attention_heads``; ``attention.head_count_kv`` ->
``num_key_value_heads``; ``attention.key_length`` -> ``head_dim``; ``feed_forward_length`` ->
``intermediate_size_mlp``; ``expert_feed_forward_length`` -> ``intermediate_size``;
``rope.freq_base`` -> ``rope_theta``; ``attention.layer_norm_rms_epsilon`` -> ``rms_norm_eps``;
``attention.sliding_window`` -> ``attention_chunk_size``; ``expert_count`` ->
``num_local_experts``; ``expert_used_count`` -> ``num_experts_per_tok``;
``interleave_moe_layer_step`` and ``vocab_size`` keep their names.

``attention_local_kind`` (this engine's own key, default ``chunk``) says what a rotating layer
reads of ``attention_chunk_size`` keys: the chunk its position lies in, or, as the reference's
forward computes it (crates/spite-models/src/llama/llama4.rs:189-197), a window of the last keys.

What the reference fixes in code is a key here: head size (``d / H`` at
crates/spite-models/src/llama/llama4.rs:87), the every-fourth-layer rule (:95), qk-norm
(:96), the temperature constants 8192 and 0.1 (:179).  The reference reads missing keys as
zero and validates nothing (config.rs:122-123); this reader reports every missing key and
every inconsistent size in one error.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a model: lists every problem found."""


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of kind ``llama3``: a per-frequency rescale applied once at load."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


@dataclass(frozen=True)
class Llama4Config:
    architecture: str
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int            # routed and shared expert width
    intermediate_size_mlp: int        # dense layers' width
    num_local_experts: int
    num_experts_per_tok: int
    interleave_moe_layer_step: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    rope_pairing: str                 # "half" (reference) or "adjacent"
    attention_chunk_size: Optional[int]
    attention_local_kind: str         # what a rotating layer reads: "chunk" (its chunk) or "window" (the last keys)
    no_rope_layers: Tuple[int, ...]   # 1 = the layer rotates (and is chunked), 0 = NoPE, full causal
    moe_layers: Tuple[int, ...]       # indices of layers with experts
    use_qk_norm: bool
    attn_temperature_tuning: bool
    floor_scale: int
    attn_scale: float
    tie_word_embeddings: bool
    max_position_embeddings: int
    torch_dtype: str
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)

    # ------------------------------------------------------------------ reading
    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "Llama4Config":
        # A multimodal checkpoint nests the text model's keys under "text_config".
        src = dict(raw.get("text_config", raw))
        problems = []

        def need(key, kind):
            if key not in src or src[key] is None:
                problems.append(f"missing key {key!r}")
                return kind()
            try:
                return kind(src[key])
            except (TypeError, ValueError):
                problems.append(f"key {key!r}: expected {kind.__name__}, got {src[key]!r}")
                return kind()

        def opt(key, kind, default):
            if key not in src or src[key] is None:
                return default
            try:
                return kind(src[key])
            except (TypeError, ValueError):
                problems.append(f"key {key!r}: expected {kind.__name__}, got {src[key]!r}")
                return default

        archs = raw.get("architectures") or src.get("architectures") or []
        if not archs:
            problems.append("missing key 'architectures'")
        arch = archs[0] if archs else ""

        L = need("num_hidden_layers", int)
        d = need("hidden_size", int)
        H = need("num_attention_heads", int)
        G = opt("num_key_value_heads", int, H)
        hd = opt("head_dim", int, d // H if H else 0)
        V = need("vocab_size", int)
        E = opt("num_local_experts", int, 0)
        k = opt("num_experts_per_tok", int, 1)
        step = opt("interleave_moe_layer_step", int, 1 if E > 0 else 0)
        F = need("intermediate_size", int) if E > 0 else opt("intermediate_size", int, 0)
        moe_layers = src.get("moe_layers")
        if moe_layers is None:
            moe_layers = [i for i in range(L) if E > 0 and step > 0 and (i + 1) % step == 0]
        moe_layers = tuple(int(i) for i in moe_layers)
        has_dense = len(set(moe_layers)) < L
        Fm = need("intermediate_size_mlp", int) if has_dense else opt("intermediate_size_mlp", int, 0)

        chunk = opt("attention_chunk_size", int, 0) or None
        nr = src.get("no_rope_layers")
        if not nr:
            interval = opt("nope_layer_interval", int, 4)
            nr = [int((i + 1) % interval != 0) for i in range(L)] if interval > 0 else [1] * L
        nr = tuple(int(bool(x)) for x in nr)

        scaling = None
        rs = src.get("rope_scaling")
        if rs:
            kind = rs.get("rope_type", rs.get("type"))
            if kind in (None, "default"):
                scaling = None
            elif kind != "llama3":
                problems.append(f"rope_scaling.rope_type {kind!r} is not supported (known: 'llama3')")
            else:
                miss = [key for key in ("factor", "low_freq_factor", "high_freq_factor",
                                        "original_max_position_embeddings") if key not in rs]
                if miss:
                    problems.append(f"rope_scaling lacks {miss}")
                else:
                    scaling = RopeScaling("llama3", float(rs["factor"]), float(rs["low_freq_factor"]),
                                          float(rs["high_freq_factor"]),
                                          int(rs["original_max_position_embeddings"]))

        eos = src.get("eos_token_id", raw.get("eos_token_id"))
        if eos is None:
            eos = ()
        elif isinstance(eos, int):
            eos = (eos,)
        else:
            eos = tuple(int(x) for x in eos)

        cfg = Llama4Config(
            architecture=arch, vocab_size=V, hidden_size=d, num_hidden_layers=L,
            num_attention_heads=H, num_key_value_heads=G, head_dim=hd,
            intermediate_size=F, intermediate_size_mlp=Fm, num_local_experts=E,
            num_experts_per_tok=k, interleave_moe_layer_step=step,
            rms_norm_eps=opt("rms_norm_eps", float, 1e-5),
            rope_theta=opt("rope_theta", float, 10000.0), rope_scaling=scaling,
            rope_pairing=opt("rope_pairing", str, "half"),
            attention_chunk_size=chunk, attention_local_kind=opt("attention_local_kind", str, "chunk"),
            no_rope_layers=nr, moe_layers=moe_layers,
            use_qk_norm=opt("use_qk_norm", bool, True),
            attn_temperature_tuning=opt("attn_temperature_tuning", bool, True),
            floor_scale=opt("floor_scale", int, 8192), attn_scale=opt("attn_scale", float, 0.1),
            tie_word_embeddings=opt("tie_word_embeddings", bool, False),
            max_position_embeddings=opt("max_position_embeddings", int, 1 << 20),
            torch_dtype=opt("torch_dtype", str, "bfloat16"),
            bos_token_id=src.get("bos_token_id"), eos_token_ids=eos)
        missing = {m.split("'")[1] for m in problems if m.startswith("missing key")}
        problems += [m for m in cfg._inconsistencies() if m.split(" ")[0] not in missing]
        if problems:
            raise ConfigError("config.json: " + "; ".join(problems))
        return cfg

    @staticmethod
    def from_json(path: str) -> "Llama4Config":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as fh:
            return Llama4Config.from_dict(json.load(fh))

    # ------------------------------------------------------------------ checking
    def _inconsistencies(self):
        p = []
        pos = dict(vocab_size=self.vocab_size, hidden_size=self.hidden_size,
                   num_hidden_layers=self.num_hidden_layers, num_attention_heads=self.num_attention_heads,
                   num_key_value_heads=self.num_key_value_heads, head_dim=self.head_dim)
        for key, val in pos.items():
            if val < 1:
                p.append(f"{key} must be >= 1, got {val}")
        if self.num_key_value_heads >= 1 and self.num_attention_heads % self.num_key_value_heads:
            p.append(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                     f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            p.append(f"head_dim {self.head_dim} must be even (rotation pairs)")
        if len(self.no_rope_layers) != self.num_hidden_layers:
            p.append(f"no_rope_layers has {len(self.no_rope_layers)} entries for "
                     f"{self.num_hidden_layers} layers")
        if self.rope_pairing not in ("half", "adjacent"):
            p.append(f"rope_pairing {self.rope_pairing!r} (known: 'half', 'adjacent')")
        if self.attention_local_kind not in ("chunk", "window"):
            p.append(f"attention_local_kind {self.attention_local_kind!r} (known: 'chunk', 'window')")
        if self.rms_norm_eps <= 0:
            p.append(f"rms_norm_eps must be > 0, got {self.rms_norm_eps}")
        if self.rope_theta <= 0:
            p.append(f"rope_theta must be > 0, got {self.rope_theta}")
        if self.attention_chunk_size is not None and self.attention_chunk_size < 1:
            p.append(f"attention_chunk_size must be >= 1, got {self.attention_chunk_size}")
        if self.moe_layers:
            if self.num_local_experts < 1:
                p.append("layers with experts need num_local_experts >= 1")
            if self.num_experts_per_tok != 1:
                p.append(f"num_experts_per_tok {self.num_experts_per_tok}: Llama 4 routes top-1")
            if self.intermediate_size < 1:
                p.append("intermediate_size must be >= 1")
            bad = [i for i in self.moe_layers if not 0 <= i < self.num_hidden_layers]
            if bad:
                p.append(f"moe_layers out of range: {bad}")
        if len(set(self.moe_layers)) < self.num_hidden_layers and self.intermediate_size_mlp < 1:
            p.append("dense layers need intermediate_size_mlp >= 1")
        if self.attn_temperature_tuning and self.floor_scale < 1:
            p.append(f"floor_scale must be >= 1, got {self.floor_scale}")
        if self.rope_scaling is not None:
            rs = self.rope_scaling
            if rs.factor <= 0 or rs.high_freq_factor <= rs.low_freq_factor or rs.original_max_position_embeddings < 1:
                p.append(f"rope_scaling is inconsistent: {rs}")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            p.append(f"torch_dtype {self.torch_dtype!r} (known: bfloat16, float32, float16)")
        return p

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = [d.pop("architecture")]
        d["no_rope_layers"] = list(self.no_rope_layers)
        d["moe_layers"] = list(self.moe_layers)
        eos = d.pop("eos_token_ids")
        if eos:
            d["eos_token_id"] = list(eos)
        if self.rope_scaling is None:
            d["rope_scaling"] = None
        if self.bos_token_id is None:
            d.pop("bos_token_id")
        d["model_type"] = "llama4_text"
        return d
