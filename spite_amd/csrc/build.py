"""Builds and loads the two native libraries of the engine.

* ``libspite_hip.so``: the gfx950 kernels (``hip/*.hip``), compiled with hipcc.
* ``libspite_host.so``: cache manager and scheduler (``host/*.cpp``), compiled with g++.

Both are built in-tree under ``csrc/_build`` (or, when the tree cannot be written, under the
user's temporary folder) the first time they are asked for and whenever a source is newer
than the library.  Nothing here imports torch; the libraries have a C interface and are
loaded with ctypes.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
GPU_ARCH = "gfx950"
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={GPU_ARCH}",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall"]

_lock = threading.Lock()
_loaded: dict = {}


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[spite_amd build] {msg}", file=sys.stderr, flush=True)


def _build_dir() -> str:
    d = os.path.join(_HERE, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"spite_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _sources(kind: str):
    sub, ext = ("hip", ".hip") if kind == "hip" else ("host", ".cpp")
    folder = os.path.join(_HERE, sub)
    srcs = sorted(os.path.join(folder, f) for f in os.listdir(folder) if f.endswith(ext))
    deps = sorted(os.path.join(folder, f) for f in os.listdir(folder) if f.endswith(".h"))
    deps.append(os.path.join(_HERE, "visibility.h"))          # shared by both libraries
    return srcs, deps


def visibility_codes() -> dict:
    """Name -> code of the rules that say which keys a query may read, as ``visibility.h``
    lists them (the header both libraries are built from is the one place that defines them)."""
    import re
    with open(os.path.join(_HERE, "visibility.h")) as f:
        m = re.search(r'#define\s+SP_VIS_NAMES\s+"([^"]*)"', f.read())
    if not m:
        raise BuildError("visibility.h does not list the rules' names")
    return {name: i for i, name in enumerate(m.group(1).split(","))}


def _find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH, /opt/rocm/bin): the HIP kernels cannot be built")


def _run(cmd, what):
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            _say(f"still compiling {what} ({time.time() - t0:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise BuildError(f"compiling {what} failed:\n{' '.join(cmd)}\n{out}")
    return out


def lib_path(kind: str) -> str:
    return os.path.join(_build_dir(), f"libspite_{kind}.so")


def is_stale(kind: str) -> bool:
    path = lib_path(kind)
    if not os.path.exists(path):
        return True
    srcs, deps = _sources(kind)
    newest = max(os.path.getmtime(p) for p in srcs + deps)
    return os.path.getmtime(path) < newest


def build(kind: str, force: bool = False) -> str:
    """Compile the library ``kind`` (``"hip"`` or ``"host"``) and return its path."""
    path = lib_path(kind)
    if not force and not is_stale(kind):
        return path
    srcs, _ = _sources(kind)
    bdir = _build_dir()
    if kind == "hip":
        cc, flags = _find_hipcc(), HIP_FLAGS
    else:
        cc = shutil.which("g++") or shutil.which("c++")
        if not cc:
            raise BuildError("no C++ compiler (g++) found for the host runtime")
        flags = HOST_FLAGS
    _say(f"compiling {len(srcs)} {kind} sources for {GPU_ARCH if kind == 'hip' else 'the host'} into {bdir}")
    t0 = time.time()
    objs = []

    def one(src):
        obj = os.path.join(bdir, f"{kind}_{os.path.basename(src)}.{os.getpid()}.o")
        _run([cc, *flags, "-c", src, "-o", obj], os.path.basename(src))
        _say(f"compiled {os.path.basename(src)} ({time.time() - t0:.0f} s)")
        return obj
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(one, srcs))
    tmp = f"{path}.{os.getpid()}.tmp"
    link = [cc, "-shared", "-fPIC", *objs, "-o", tmp]
    if kind == "hip":
        link.insert(1, f"--offload-arch={GPU_ARCH}")
    _run(link, f"libspite_{kind}.so (link)")
    os.replace(tmp, path)
    for o in objs:
        try:
            os.remove(o)
        except OSError:
            pass
    _say(f"built {os.path.basename(path)} in {time.time() - t0:.0f} s")
    return path


def load(kind: str) -> ctypes.CDLL:
    """The library, built first if it is missing or older than its sources."""
    with _lock:
        if kind in _loaded:
            return _loaded[kind]
        path = build(kind)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from e
        _loaded[kind] = lib
        return lib


def build_all(force: bool = True) -> None:
    for kind in ("host", "hip"):
        build(kind, force=force)
