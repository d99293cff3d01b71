"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

Every tensor is drawn from its own generator, seeded by (seed, crc32 of the tensor's name),
so the numbers do not depend on the order of the tensors.  Matrices are N(0, std); norm
weights 1 + N(0, std) (weights near zero would scale every activation down to where
attention is uniform and every logit near a tie).  The choice is recorded in config.json
under ``spite_random_init``.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict

import torch

from ..config import read_config
from ..engine.context import Env
from .safetensors_io import write_safetensors

_FILE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


def draw(name: str, spec, seed: int, std: float) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode())) % (1 << 63))
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32)
    t = torch.randn(spec.shape, generator=g, dtype=torch.float32) * std
    return t + 1.0 if spec.init == "ones" else t


def random_tensors(config: dict, seed: int, std: float = 0.02) -> Dict[str, torch.Tensor]:
    """fp32 tensors by checkpoint name for ``config`` (a config.json dict)."""
    from ..engine.model import Model
    arch, cfg = read_config(config)
    model = Model(arch.build_spec(cfg), Env(torch.float32, torch.device("cpu")))
    out = {}
    for fname, ps, _, _ in model.tensor_plan():
        if fname not in out:
            out[fname] = draw(fname, ps, seed, std)
    return out


def write_random_model(folder: str, config: dict, seed: int, std: float = 0.02, dtype: str | None = None,
                       overrides: Dict[str, torch.Tensor] | None = None) -> str:
    """Writes ``folder/config.json`` and ``folder/model.safetensors``; returns the folder.

    ``dtype`` of the stored matrices defaults to the config's ``torch_dtype``.  ``overrides``
    replaces tensors by name (tests plant special weights this way)."""
    config = dict(config)
    dtype = dtype or config.get("torch_dtype", "bfloat16")
    if dtype not in _FILE_DTYPES:
        raise ValueError(f"dtype {dtype!r} (known: {sorted(_FILE_DTYPES)})")
    config["torch_dtype"] = dtype
    tensors = random_tensors(config, seed, std)
    for name, t in (overrides or {}).items():
        if name not in tensors:
            raise KeyError(f"override for unknown tensor {name!r}")
        if tuple(t.shape) != tuple(tensors[name].shape):
            raise ValueError(f"override for {name}: shape {tuple(t.shape)}, expected {tuple(tensors[name].shape)}")
        tensors[name] = t.to(torch.float32) if t.is_floating_point() else t
    stored = {n: (t.to(_FILE_DTYPES[dtype]) if t.is_floating_point() else t) for n, t in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    config["spite_random_init"] = {"seed": int(seed), "std": float(std), "matrices": "N(0,std)",
                                   "norm_weights": "1+N(0,std)"}
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config, fh, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), stored, {"format": "pt"})
    return folder
