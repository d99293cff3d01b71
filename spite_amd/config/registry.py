"""One registry from an architecture's name (``architectures[0]`` of config.json) to its
typed configuration and the function that turns it into a ``ModelSpec``.

The reference keeps a list of (name, constructor) pairs and answers an unknown name with
``UnknownArch`` (crates/spite-models/src/lib.rs:386-436); so does this one, listing the
names it knows.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict


class UnknownArchitecture(KeyError):
    pass


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[dict], Any]
    build_spec: Callable[[Any], Any]          # config -> parts.ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, build_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_from_dict, build_spec)


def architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise UnknownArchitecture(
            f"unknown architecture {name!r}; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def registered_architectures():
    return sorted(_ARCHITECTURES)


def read_config(source):
    """(Architecture, typed config) from a model folder, a config.json path or a dict."""
    if isinstance(source, dict):
        raw = source
    else:
        path = os.path.join(source, "config.json") if os.path.isdir(source) else source
        with open(path, "r", encoding="utf-8") as fh:
            raw = json.load(fh)
    archs = raw.get("architectures") or raw.get("text_config", {}).get("architectures") or []
    if not archs:
        raise UnknownArchitecture(f"config names no architecture; registered: {sorted(_ARCHITECTURES)}")
    arch = architecture(archs[0])
    return arch, arch.config_from_dict(raw)
