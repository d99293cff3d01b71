"""Random-weights mode: writes a model folder (config.json, model.safetensors) from a
configuration and a seed.

Element i of a tensor is a function of (seed, crc32 of the tensor's name, i) alone, so the
numbers do not depend on the order of drawing, and the engine's own random-weights mode, which
draws on the GPU, holds the model that the folder of the same seed holds.  Matrices are N(0, std); norm
weights 1 + N(0, std) (weights near zero would scale every activation down to where
attention is uniform and every logit near a tie).  The choice is recorded in config.json
under ``spite_random_init``.
"""
from __future__ import annotations

import json
import os
import zlib
from concurrent.futures import ThreadPoolExecutor
from typing import Dict

import numpy as np
import torch

from ..config import read_config
from ..engine.context import Env
from .safetensors_io import write_safetensors

_FILE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


_M64 = (1 << 64) - 1


def _mix64(x: np.ndarray) -> np.ndarray:
    x = x ^ (x >> np.uint64(30))
    x = x * np.uint64(0xbf58476d1ce4e5b9)
    x = x ^ (x >> np.uint64(27))
    x = x * np.uint64(0x94d049bb133111eb)
    return x ^ (x >> np.uint64(31))


def _exact_log(x: np.ndarray) -> np.ndarray:
    m, e = np.frexp(x)
    small = m < 0.70710678118654752
    m = np.where(small, m * 2.0, m)
    e = np.where(small, e - 1, e)
    s = (m - 1.0) / (m + 1.0)
    s2 = s * s
    p = np.full_like(s, 1.0 / 23.0)
    for k in (21.0, 19.0, 17.0, 15.0, 13.0, 11.0, 9.0, 7.0, 5.0, 3.0):
        p = p * s2 + 1.0 / k
    p = p * s2 + 1.0
    return e.astype(np.float64) * 0.6931471805599453 + 2.0 * (s * p)


def _exact_sincos_turns(k: np.ndarray):
    quad = k >> np.uint32(30)
    low = k & np.uint32(0x3fffffff)
    fold = low > np.uint32(0x20000000)
    a = np.where(fold, np.uint32(0x40000000) - low, low)
    t = a.astype(np.float64) * (1.5707963267948966 / 1073741824.0)
    t2 = t * t
    ps = np.full_like(t, 1.0 / 355687428096000.0)
    for sign, f in ((-1, 1307674368000.0), (1, 6227020800.0), (-1, 39916800.0), (1, 362880.0), (-1, 5040.0),
                    (1, 120.0), (-1, 6.0)):
        ps = ps * t2 + 1.0 / f if sign > 0 else ps * t2 - 1.0 / f
    ps = ps * t2 + 1.0
    pc = np.full_like(t, -1.0 / 6402373705728000.0)
    for sign, f in ((1, 20922789888000.0), (-1, 87178291200.0), (1, 479001600.0), (-1, 3628800.0), (1, 40320.0),
                    (-1, 720.0), (1, 24.0), (-1, 2.0)):
        pc = pc * t2 + 1.0 / f if sign > 0 else pc * t2 - 1.0 / f
    pc = pc * t2 + 1.0
    tps = t * ps
    s0 = np.where(fold, pc, tps)
    c0 = np.where(fold, tps, pc)
    sn = np.select([quad == 0, quad == 1, quad == 2], [s0, c0, -s0], -c0)
    cs = np.select([quad == 0, quad == 1, quad == 2], [c0, -s0, -c0], s0)
    return sn, cs


def normal_numbers(n: int, seed: int, key: int, mean: float = 0.0, std: float = 1.0) -> np.ndarray:
    """float32 [n]: the numbers that the kernel ``randn_fill`` writes for (seed, key), bit for bit.
    Element i depends on (seed, key, i) alone.  A 64-bit mix of (seed, key, i // 2) gives two
    uniform numbers of 32 bits; Box-Muller turns them into the normals of elements i and i + 1;
    logarithm, sine and cosine are sums of IEEE double operations in a fixed order (the kernel
    forms the same sums without fused multiply-adds), so both sides round alike."""
    base = (int(seed) * 0x9e3779b97f4a7c15 + int(key)) & _M64
    out = np.empty(n, dtype=np.float32)
    pairs = (n + 1) // 2
    step = 1 << 18
    with np.errstate(over="ignore"):
        base = _mix64(np.array([base], dtype=np.uint64))[0]

    def block(j0):
        with np.errstate(over="ignore"):
            j = np.arange(j0, min(j0 + step, pairs), dtype=np.uint64)
            h = _mix64(base + j * np.uint64(0xd1342543de82ef95))
        u1 = ((h >> np.uint64(32)).astype(np.float64) + 1.0) * (1.0 / 4294967296.0)
        r = np.sqrt(-2.0 * _exact_log(u1))
        sn, cs = _exact_sincos_turns((h & np.uint64(0xffffffff)).astype(np.uint32))
        both = np.empty(2 * len(j), dtype=np.float32)
        both[0::2] = np.float32(std) * (r * cs).astype(np.float32) + np.float32(mean)
        both[1::2] = np.float32(std) * (r * sn).astype(np.float32) + np.float32(mean)
        out[2 * j0:2 * j0 + min(2 * len(j), n - 2 * j0)] = both[:n - 2 * j0]

    starts = range(0, pairs, step)
    if len(starts) > 1:          # numpy's loops release the interpreter's lock: blocks run side by side
        with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            list(pool.map(block, starts))
    else:
        for j0 in starts:
            block(j0)
    return out


def tensor_key(name: str) -> int:
    return zlib.crc32(name.encode())


def draw(name: str, spec, seed: int, std: float) -> torch.Tensor:
    """The tensor ``name`` of a random model, on the host, fp32 (int32 tables are zero)."""
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32)
    n = 1
    for s in spec.shape:
        n *= int(s)
    z = normal_numbers(n, seed, tensor_key(name), 1.0 if spec.init == "ones" else 0.0, std)
    return torch.from_numpy(z).view(tuple(spec.shape))


def draw_on_device(name: str, spec, seed: int, std: float, file_dtype: torch.dtype, device) -> torch.Tensor:
    """The same tensor drawn by the kernel on the GPU, rounded to ``file_dtype`` as the folder
    of that seed stores it."""
    from ..csrc import hipops
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    direct = file_dtype in (torch.float32, torch.bfloat16)
    t = torch.empty(spec.shape, dtype=file_dtype if direct else torch.float32, device=device)
    if spec.init == "zeros":
        t.zero_()
    else:
        hipops.randn_fill(t, seed, tensor_key(name), 1.0 if spec.init == "ones" else 0.0, std)
    return t if direct else t.to(file_dtype)


def random_tensors(config: dict, seed: int, std: float = 0.02, device=None) -> Dict[str, torch.Tensor]:
    """fp32 tensors by checkpoint name for ``config`` (a config.json dict), on the host.  With a
    GPU ``device`` they are drawn there and copied back: the same numbers, sooner."""
    from ..engine.model import Model
    arch, cfg = read_config(config)
    model = Model(arch.build_spec(cfg), Env(torch.float32, torch.device("cpu")))
    out = {}
    for fname, ps, _, _ in model.tensor_plan():
        if fname not in out:
            out[fname] = draw(fname, ps, seed, std) if device is None else \
                draw_on_device(fname, ps, seed, std, torch.float32, device).cpu()
    return out


def write_random_model(folder: str, config: dict, seed: int, std: float = 0.02, dtype: str | None = None,
                       overrides: Dict[str, torch.Tensor] | None = None, device=None, keep_wide=()) -> str:
    """Writes ``folder/config.json`` and ``folder/model.safetensors``; returns the folder.

    ``dtype`` of the stored matrices defaults to the config's ``torch_dtype``.  ``overrides``
    replaces tensors by name (tests plant special weights this way).  ``keep_wide``: substrings of
    tensor names that are stored in float32 whatever ``dtype`` is (a checkpoint that keeps some
    of its tensors in 32-bit beside bfloat16 ones)."""
    config = dict(config)
    dtype = dtype or config.get("torch_dtype", "bfloat16")
    if dtype not in _FILE_DTYPES:
        raise ValueError(f"dtype {dtype!r} (known: {sorted(_FILE_DTYPES)})")
    config["torch_dtype"] = dtype
    tensors = random_tensors(config, seed, std, device)
    for name, t in (overrides or {}).items():
        if name not in tensors:
            raise KeyError(f"override for unknown tensor {name!r}")
        if tuple(t.shape) != tuple(tensors[name].shape):
            raise ValueError(f"override for {name}: shape {tuple(t.shape)}, expected {tuple(tensors[name].shape)}")
        tensors[name] = t.to(torch.float32) if t.is_floating_point() else t
    wide = lambda n: any(k in n for k in keep_wide)
    stored = {n: (t.to(torch.float32 if wide(n) else _FILE_DTYPES[dtype]) if t.is_floating_point() else t)
              for n, t in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    config["spite_random_init"] = {"seed": int(seed), "std": float(std), "matrices": "N(0,std)",
                                   "norm_weights": "1+N(0,std)"}
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config, fh, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), stored, {"format": "pt"})
    return folder
