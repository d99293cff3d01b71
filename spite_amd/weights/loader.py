"""Binds the tensors of a checkpoint to the parts of a model, by name.

Every problem is found before anything is moved to the GPU and reported in one
``WeightsError``: tensors the model needs and the file lacks, tensors of the file that the
model does not know, wrong shapes, integer tables stored as floats (or the reverse).
The tensors come from a source: a model folder, a dict in memory, or a seed; all three go
through the same check and the same binding (``bind``).

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


def _strip(name: str, prefixes=PREFIXES) -> str:
    for p in prefixes:
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


class FolderSource:
    """The tensors of a model folder (``model.safetensors`` or its shards)."""

    def __init__(self, folder: str, strip=PREFIXES, ignore=()):
        self.where = folder
        self._ckpt = Checkpoint(folder)
        self._have: Dict[str, str] = {}
        for name in self._ckpt.names():
            if any(name.startswith(p) for p in ignore):
                continue
            self._have[_strip(name, strip)] = name

    def names(self):
        return list(self._have)

    def info(self, name):
        return self._ckpt.info(self._have[name])

    def host(self, name) -> torch.Tensor:
        return self._ckpt.tensor(self._have[name])

    def on_device(self, name, spec, device, dtype) -> torch.Tensor:
        return self.host(name).to(device=device, dtype=dtype)


class DictSource:
    """Tensors handed over in memory, by checkpoint name."""

    def __init__(self, tensors: Dict[str, torch.Tensor]):
        self.where = "the given tensors"
        self._t = tensors

    def names(self):
        return list(self._t)

    def info(self, name):
        return self._t[name].dtype, tuple(self._t[name].shape)

    def host(self, name) -> torch.Tensor:
        return self._t[name].detach().cpu()

    def on_device(self, name, spec, device, dtype) -> torch.Tensor:
        return self._t[name].to(device=device, dtype=dtype)


class RandomSource:
    """Every tensor of the plan drawn from a seed (``random_init.draw``): on the GPU when the
    model is bound, on the host when a tensor is read back, the same numbers either way, and the
    numbers that the random-weights folder of that seed holds.  ``file_dtype``: the dtype such
    a folder stores floating tensors in; the drawn numbers are rounded to it first."""

    def __init__(self, plan, seed: int, std: float, file_dtype: torch.dtype):
        self.where = f"random weights of seed {seed}"
        self.seed, self.std, self.file_dtype = int(seed), float(std), file_dtype
        self._specs = {}
        for fname, ps, _, _ in plan:
            self._specs.setdefault(fname, ps)

    def names(self):
        return list(self._specs)

    def info(self, name):
        ps = self._specs[name]
        return (torch.int32 if ps.kind == "int" else self.file_dtype), tuple(ps.shape)

    def host(self, name) -> torch.Tensor:
        from .random_init import draw
        t = draw(name, self._specs[name], self.seed, self.std)
        return t.to(self.file_dtype) if t.is_floating_point() else t

    def on_device(self, name, spec, device, dtype) -> torch.Tensor:
        from .random_init import draw_on_device
        return draw_on_device(name, spec, self.seed, self.std, self.file_dtype, device).to(dtype)


def bind(model, source, checkpoint_dtype: torch.dtype = torch.bfloat16) -> None:
    """Checks the model's tensor plan against ``source`` (one error for everything that does
    not fit), then hands every part its tensors on the GPU in their resident dtype."""
    plan = model.tensor_plan()
    have = set(source.names())
    expected = {}
    for fname, ps, owner, local in plan:
        expected.setdefault(fname, (ps, owner, local))
    missing = [n for n in expected if n not in have]
    unexpected = [n for n in have if n not in expected]
    shapes, kinds = [], []
    for n, (ps, _, _) in expected.items():
        if n not in have:
            continue
        dt, shape = source.info(n)
        if tuple(shape) != tuple(ps.shape):
            shapes.append((n, shape, ps.shape))
        is_int = not dt.is_floating_point
        if (ps.kind == "int") != is_int:
            kinds.append((n, dt, "an integer type" if ps.kind == "int" else "a floating type"))
    if missing or unexpected or shapes or kinds:
        raise WeightsError(sorted(missing), sorted(unexpected), shapes, kinds, source.where)

    run_dtype, device = model.env.dtype, model.env.device
    by_owner: Dict[int, tuple] = {}
    for fname, ps, owner, local in plan:
        by_owner.setdefault(id(owner), (owner, {}))[1][local] = (fname, ps)
    for owner, locs in by_owner.values():
        tensors = {}
        for local, (fname, ps) in locs.items():
            stored, _ = source.info(fname)
            tensors[local] = source.on_device(fname, ps, device, resident_dtype(stored, ps.kind, run_dtype, checkpoint_dtype))
        owner.load(tensors)
        tensors.clear()
    model.finish_loading()


def load_weights(model, folder: str, checkpoint_dtype: torch.dtype = torch.bfloat16) -> None:
    spec = model.spec
    bind(model, FolderSource(folder, getattr(spec, "strip_prefixes", PREFIXES), getattr(spec, "ignore_prefixes", ())),
         checkpoint_dtype)
