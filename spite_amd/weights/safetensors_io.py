"""Reader and writer of the safetensors container: 8 bytes little-endian header length, a
JSON header ``{name: {dtype, shape, data_offsets}}``, then the raw data.

The reader maps the file and hands out tensors that view the mapping (no copy until they
are moved to the GPU).  A folder may hold one ``model.safetensors`` or several shards with a
``model.safetensors.index.json``.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, Tuple

import torch

DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
NAMES = {v: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: {size} bytes is too short for a safetensors file")
        self._fh = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._fh.read(8))
        if hlen > size - 8 or hlen > (100 << 20):
            raise SafetensorsError(f"{path}: header length {hlen} does not fit the file of {size} bytes")
        try:
            header = json.loads(self._fh.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from e
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + hlen
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        data_len = size - self._data_start
        for name, info in header.items():
            try:
                dt, shape, (b, e) = info["dtype"], tuple(int(x) for x in info["shape"]), info["data_offsets"]
            except (KeyError, TypeError, ValueError) as ex:
                raise SafetensorsError(f"{path}: malformed entry for {name!r}") from ex
            if dt not in DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt}")
            numel = 1
            for s in shape:
                numel *= s
            want = numel * torch.empty((), dtype=DTYPES[dt]).element_size()
            if b < 0 or e < b or e > data_len or e - b != want:
                raise SafetensorsError(
                    f"{path}: tensor {name!r} ({dt}{list(shape)}) claims bytes [{b},{e}) of {data_len}: truncated or corrupt")
            self.entries[name] = (dt, shape, b, e)
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ) if size > 0 else None

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def info(self, name: str):
        dt, shape, _, _ = self.entries[name]
        return DTYPES[dt], shape

    def tensor(self, name: str) -> torch.Tensor:
        dt, shape, b, e = self.entries[name]
        if e == b:
            return torch.empty(shape, dtype=DTYPES[dt])
        buf = memoryview(self._mm)[self._data_start + b:self._data_start + e]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")      # the mapping is read-only; tensors are only read
            t = torch.frombuffer(buf, dtype=DTYPES[dt])
        return t.view(shape)


class Checkpoint:
    """All tensors of a model folder, by name."""

    def __init__(self, folder: str):
        self.folder = folder
        index = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.exists(index):
            with open(index, "r", encoding="utf-8") as fh:
                wm = json.load(fh).get("weight_map", {})
            for name, fname in wm.items():
                self._where[name] = fname
            for fname in sorted(set(wm.values())):
                self._files[fname] = SafetensorsFile(os.path.join(folder, fname))
        elif os.path.exists(single):
            f = SafetensorsFile(single)
            self._files["model.safetensors"] = f
            for name in f.names():
                self._where[name] = "model.safetensors"
        else:
            raise SafetensorsError(f"{folder}: no model.safetensors (or model.safetensors.index.json)")

    def names(self):
        return list(self._where.keys())

    def info(self, name):
        return self._files[self._where[name]].info(name)

    def tensor(self, name):
        return self._files[self._where[name]].tensor(name)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] | None = None) -> None:
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    off = 0
    order = sorted(tensors.keys())
    for name in order:
        t = tensors[name]
        if t.dtype not in NAMES:
            raise SafetensorsError(f"cannot store dtype {t.dtype} ({name})")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + n]}
        off += n
    hj = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hj += b" " * ((8 - len(hj) % 8) % 8)
    tmp = f"{path}.tmp{os.getpid()}"
    with open(tmp, "wb") as fh:
        fh.write(struct.pack("<Q", len(hj)))
        fh.write(hj)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            fh.write(t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
