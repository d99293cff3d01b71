"""Weights: the safetensors container, binding by name with one error for everything that
does not fit, resident dtypes, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B
from spite_amd.config import read_config
from spite_amd.engine.context import Env
from spite_amd.engine.model import Model
from spite_amd.weights.loader import load_weights, WeightsError, resident_dtype
from spite_amd.weights.random_init import write_random_model, random_tensors
from spite_amd.weights.safetensors_io import (SafetensorsFile, SafetensorsError, Checkpoint, write_safetensors)


def cpu_model(cfg, dtype=torch.float32):
    arch, c = read_config(cfg)
    return Model(arch.build_spec(c), Env(dtype, torch.device("cpu")))


def test_container_round_trip_against_the_library(tmp_path):
    t = {"a": torch.randn(3, 5), "b.c": torch.randn(7).to(torch.bfloat16), "n": torch.arange(6, dtype=torch.int32).view(2, 3)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, t, {"format": "pt"})
    lib = load_file(p)                                     # the library reads what we wrote
    for k in t:
        assert torch.equal(lib[k], t[k])
    p2 = str(tmp_path / "y.safetensors")
    save_file(t, p2)
    mine = SafetensorsFile(p2)                             # and we read what the library wrote
    assert sorted(mine.names()) == sorted(t)
    for k in t:
        assert torch.equal(mine.tensor(k), t[k]) and mine.info(k) == (t[k].dtype, tuple(t[k].shape))


def test_container_errors(tmp_path):
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, {"a": torch.randn(4, 4)})
    raw = open(p, "rb").read()
    open(p, "wb").write(raw[:-8])
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(SafetensorsError, match="JSON"):
        SafetensorsFile(p)
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        Checkpoint(str(tmp_path / "empty"))


def test_random_model_folder(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_B, seed=11)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    cfg = json.load(open(os.path.join(d, "config.json")))
    assert cfg["spite_random_init"]["seed"] == 11 and cfg["hidden_size"] == 96
    w = load_file(os.path.join(d, "model.safetensors"))
    assert w["model.layers.1.feed_forward.experts.gate_up_proj"].shape == (8, 96, 128)
    assert w["model.layers.1.feed_forward.experts.down_proj"].shape == (8, 64, 96)
    assert w["model.layers.0.feed_forward.gate_proj.weight"].shape == (192, 96)
    assert w["model.layers.0.self_attn.q_proj.weight"].shape == (6 * 24, 96)
    assert w["model.layers.0.self_attn.k_proj.weight"].shape == (3 * 24, 96)
    assert "model.layers.0.feed_forward.router.weight" not in w and "model.layers.1.feed_forward.router.weight" in w
    assert abs(float(w["model.norm.weight"].mean()) - 1.0) < 0.05            # norm weights around one
    assert abs(float(w["lm_head.weight"].std()) - 0.02) < 0.003
    # same seed, same numbers; another seed, others; a tensor's numbers do not depend on the rest
    again = random_tensors(TINY_B, 11)
    assert torch.equal(again["lm_head.weight"], w["lm_head.weight"])
    assert not torch.equal(random_tensors(TINY_B, 12)["lm_head.weight"], w["lm_head.weight"])
    fewer = random_tensors(dict(TINY_B, num_hidden_layers=4), 11)
    assert torch.equal(fewer["model.layers.3.self_attn.o_proj.weight"], w["model.layers.3.self_attn.o_proj.weight"])


def test_loading_binds_every_tensor(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=3)
    m = cpu_model(TINY_A)
    load_weights(m, d, torch.float32)
    w = load_file(os.path.join(d, "model.safetensors"))
    assert torch.equal(m.embedding.table, w["model.embed_tokens.weight"]) and torch.equal(m.head.weight.data, w["lm_head.weight"])
    att = m.blocks[2].mixer
    assert not att.wqkv.tiled                     # operand order is for bfloat16 matrices on the GPU
    assert torch.equal(att.wqkv.data[:64], w["model.layers.2.self_attn.q_proj.weight"])
    assert torch.equal(att.wqkv.data[64:96], w["model.layers.2.self_attn.k_proj.weight"])
    ffn = m.blocks[2].ffn
    gu = w["model.layers.2.feed_forward.experts.gate_up_proj"]              # [E, d, 2F]
    assert ffn.w_gate_up.shape == (5, 256, 64)                               # experts + shared, rows gate then up
    wgu, wdn = ffn.w_gate_up.data, ffn.w_down.data
    assert torch.equal(wgu[1, :128], gu[1, :, :128].T) and torch.equal(wgu[1, 128:], gu[1, :, 128:].T)
    assert torch.equal(wgu[4, :128], w["model.layers.2.feed_forward.shared_expert.gate_proj.weight"])
    assert torch.equal(wdn[3], w["model.layers.2.feed_forward.experts.down_proj"][3].T)
    assert torch.equal(wdn[4], w["model.layers.2.feed_forward.shared_expert.down_proj.weight"])


def test_operand_order_puts_each_lanes_eight_elements_where_the_kernels_read_them():
    from spite_amd.csrc.hipops import operand_order, KernelError
    N, K = 48, 128
    w = torch.arange(2 * N * K, dtype=torch.float32).view(2, N, K)
    t = operand_order(w).reshape(2, -1)
    for g, n, k in [(0, 0, 0), (0, 17, 33), (1, 47, 127), (1, 16, 64), (0, 31, 95)]:
        i, r, j, q, e = n // 16, n % 16, k // 32, (k % 32) // 8, k % 8
        at = ((i * (K // 32)) + j) * 512 + (q * 16 + r) * 8 + e
        assert t[g, at] == w[g, n, k]
    with pytest.raises(KernelError):
        operand_order(torch.zeros(24, 64))
    with pytest.raises(KernelError):
        operand_order(torch.zeros(32, 96))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=3)
    p = os.path.join(d, "model.safetensors")
    w = load_file(p)
    del w["model.layers.1.self_attn.o_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.9.extra.weight"] = torch.zeros(2)
    w["lm_head.weight"] = torch.zeros(255, 64)
    w["model.layers.0.feed_forward.router.weight"] = torch.zeros(4, 64, dtype=torch.int32)
    save_file(w, p)
    with pytest.raises(WeightsError) as e:
        load_weights(cpu_model(TINY_A), d, torch.float32)
    err = e.value
    assert err.missing == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.9.extra.weight"]
    assert err.shapes == [("lm_head.weight", (255, 64), (256, 64))]
    assert [k[0] for k in err.kinds] == ["model.layers.0.feed_forward.router.weight"]
    msg = str(err)
    for piece in ("missing tensors", "unexpected tensors", "wrong shapes", "[255, 64], expected [256, 64]", "wrong dtypes"):
        assert piece in msg, msg


def test_language_model_prefix_is_stripped(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=3)
    p = os.path.join(d, "model.safetensors")
    save_file({"language_model." + k: v for k, v in load_file(p).items()}, p)
    load_weights(cpu_model(TINY_A), d, torch.float32)


def test_tied_embeddings_need_no_head(tmp_path):
    cfg = dict(TINY_A, tie_word_embeddings=True)
    d = write_random_model(str(tmp_path / "m"), cfg, seed=3)
    assert "lm_head.weight" not in load_file(os.path.join(d, "model.safetensors"))
    m = cpu_model(cfg)
    load_weights(m, d, torch.float32)
    assert m.head.weight is m.embedding.table


def test_resident_dtypes():
    bf, f32 = torch.bfloat16, torch.float32
    assert resident_dtype(bf, "matrix", bf, bf) == bf
    assert resident_dtype(f32, "matrix", bf, bf) == f32        # stored in 32-bit by a 16-bit checkpoint: stays
    assert resident_dtype(f32, "matrix", bf, f32) == bf        # a 32-bit checkpoint run in bfloat16
    assert resident_dtype(bf, "matrix", f32, bf) == f32        # a float32 run widens everything
    assert resident_dtype(bf, "vector", bf, bf) == f32         # norm weights and router in 32-bit
    assert resident_dtype(torch.int64, "int", bf, bf) == torch.int32


def test_mixed_checkpoint_keeps_32_bit_tensors(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=3, dtype="bfloat16")
    p = os.path.join(d, "model.safetensors")
    w = load_file(p)
    w["model.layers.0.self_attn.o_proj.weight"] = w["model.layers.0.self_attn.o_proj.weight"].float()
    save_file(w, p)
    m = cpu_model(TINY_A, torch.bfloat16)
    load_weights(m, d, torch.bfloat16)
    assert m.blocks[0].mixer.wo.dtype == torch.float32 and m.blocks[1].mixer.wo.dtype == torch.bfloat16
    assert m.blocks[0].norm1.weight.dtype == torch.float32 and m.blocks[0].ffn.w_router.dtype == torch.float32
    assert m.embedding.table.dtype == torch.bfloat16


def test_text_model_of_a_multimodal_folder(tmp_path):
    # keys under text_config, tensors under language_model., other towers' tensors passed over;
    # an unknown tensor under the text prefix is still an error, and so is a tower's tensor in a
    # folder that says it is a text model
    from spite_amd.weights.random_init import random_tensors
    text = {k: v for k, v in TINY_A.items() if k != "architectures"}
    cfg = {"architectures": ["Llama4ForConditionalGeneration"], "text_config": text}
    d = str(tmp_path / "mm")
    os.makedirs(d)
    json.dump(cfg, open(os.path.join(d, "config.json"), "w"))
    t = {"language_model." + k: v for k, v in random_tensors(TINY_A, 3).items()}
    t["vision_model.patch_embedding.weight"] = torch.zeros(4, 4)
    t["multi_modal_projector.linear_1.weight"] = torch.zeros(2, 2)
    save_file(t, os.path.join(d, "model.safetensors"))
    arch, c = read_config(d)
    assert arch.name == "Llama4ForConditionalGeneration" and c.hidden_size == TINY_A["hidden_size"]
    m = Model(arch.build_spec(c), Env(torch.float32, torch.device("cpu")))
    load_weights(m, d, torch.float32)
    assert m.embedding.table.shape == (TINY_A["vocab_size"], TINY_A["hidden_size"])
    t["language_model.model.layers.0.extra.weight"] = torch.zeros(1)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError, match="unexpected tensors: model.layers.0.extra.weight") as e:
        load_weights(m, d, torch.float32)
    assert "vision_model" not in str(e.value)
    with pytest.raises(WeightsError, match="vision_model"):
        load_weights(cpu_model(TINY_A), d, torch.float32)


def test_one_binder_for_folders_tensors_in_memory_and_seeds():
    from spite_amd.weights.loader import bind, DictSource, RandomSource
    from spite_amd.weights.random_init import random_tensors, draw
    m = cpu_model(TINY_B)
    t = random_tensors(TINY_B, 9)
    src = RandomSource(m.tensor_plan(), 9, 0.02, torch.float32)
    assert sorted(src.names()) == sorted(t)
    for n in t:
        assert torch.equal(src.host(n), t[n])
    bad = dict(t)
    bad.pop("model.norm.weight")
    bad["lm_head.weight"] = bad["lm_head.weight"][:-1]
    bad["stray"] = torch.zeros(1)
    with pytest.raises(WeightsError) as e:
        bind(m, DictSource(bad), torch.float32)
    msg = str(e.value)
    assert "missing tensors: model.norm.weight" in msg and "unexpected tensors: stray" in msg and "lm_head.weight is" in msg
    bind(m, DictSource(t), torch.float32)
    assert torch.equal(m.final_norm.weight, t["model.norm.weight"])
