"""Binds the tensors of a checkpoint to the parts of a model, by name.

Every problem is found before anything is moved to the GPU and reported in one
``WeightsError``: tensors the model needs and the file lacks, tensors of the file that the
model does not know, wrong shapes, integer tables stored as floats (or the reverse).

Resident dtypes: "vector" tensors (norm weights, router) are fp32; "int" tensors int32;
"matrix" tensors take the run's dtype, except that in a bfloat16 run a matrix that the
checkpoint stores in 32-bit although its ``torch_dtype`` is 16-bit stays in 32-bit.  In a
float32 run everything is widened to fp32.
"""
from __future__ import annotations

from typing import Dict

import torch

from .safetensors_io import Checkpoint

PREFIXES = ("language_model.",)


class WeightsError(ValueError):
    def __init__(self, missing=(), unexpected=(), shapes=(), kinds=(), folder=""):
        self.missing, self.unexpected, self.shapes, self.kinds = list(missing), list(unexpected), list(shapes), list(kinds)

        def some(xs):
            xs = list(xs)
            return ", ".join(xs[:12]) + (f", ... ({len(xs)} in all)" if len(xs) > 12 else "")
        parts = []
        if self.missing:
            parts.append(f"missing tensors: {some(self.missing)}")
        if self.unexpected:
            parts.append(f"unexpected tensors: {some(self.unexpected)}")
        if self.shapes:
            parts.append("wrong shapes: " + some(f"{n} is {list(a)}, expected {list(e)}" for n, a, e in self.shapes))
        if self.kinds:
            parts.append("wrong dtypes: " + some(f"{n} is {a}, expected {e}" for n, a, e in self.kinds))
        super().__init__(f"weights of {folder or 'the model'} do not fit: " + "; ".join(parts))


def _strip(name: str) -> str:
    for p in PREFIXES:
        if name.startswith(p):
            return name[len(p):]
    return name


def resident_dtype(stored: torch.dtype, kind: str, run_dtype: torch.dtype, checkpoint_dtype: torch.dtype):
    if kind == "int":
        return torch.int32
    if kind == "vector" or run_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64) and checkpoint_dtype != torch.float32:
        return torch.float32          # deliberately kept wide by the checkpoint
    return run_dtype


def load_weights(model, folder: str, checkpoint_dtype: torch.dtype = torch.bfloat16) -> None:
    ckpt = Checkpoint(folder)
    have: Dict[str, str] = {}
    for name in ckpt.names():
        have[_strip(name)] = name
    plan = model.tensor_plan()
    expected = {}
    for fname, ps, owner, local in plan:
        expected.setdefault(fname, (ps, owner, local))
    missing = [n for n in expected if n not in have]
    unexpected = [n for n in have if n not in expected]
    shapes, kinds = [], []
    for n, (ps, _, _) in expected.items():
        if n not in have:
            continue
        dt, shape = ckpt.info(have[n])
        if tuple(shape) != tuple(ps.shape):
            shapes.append((n, shape, ps.shape))
        is_int = not dt.is_floating_point
        if (ps.kind == "int") != is_int:
            kinds.append((n, dt, "an integer type" if ps.kind == "int" else "a floating type"))
    if missing or unexpected or shapes or kinds:
        raise WeightsError(sorted(missing), sorted(unexpected), shapes, kinds, folder)

    run_dtype, device = model.env.dtype, model.env.device
    by_owner: Dict[int, tuple] = {}
    for fname, ps, owner, local in plan:
        by_owner.setdefault(id(owner), (owner, {}))[1][local] = (fname, ps)
    for owner, locs in by_owner.values():
        tensors = {}
        for local, (fname, ps) in locs.items():
            t = ckpt.tensor(have[fname])
            tensors[local] = t.to(device=device, dtype=resident_dtype(t.dtype, ps.kind, run_dtype, checkpoint_dtype))
        owner.load(tensors)
    model.finish_loading()
