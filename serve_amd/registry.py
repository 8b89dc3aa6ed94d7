"""Registries: architecture name -> (configuration class, spec builder) and part kind -> class.

`architectures[0]` of config.json selects the architecture, as the reference's
`name_to_config[model_name]` does for its two models (serve/utils.py:35-38,54).  Part kinds
(`mixer`, `feed_forward`, `norm`, `position`, `embedding`, `lm_head`, `arrangement`) are
looked up when a `ModelSpec` is built into a model, so a new part is one `register_part`
call and needs no change to the model, engine, cache or scheduler.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Tuple


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]
    build_spec: Callable[[Any], Any]          # typed config -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}
_PARTS: Dict[Tuple[str, str], type] = {}

PART_ROLES = ("mixer", "feed_forward", "norm", "position", "embedding", "lm_head", "arrangement")


def register_architecture(name: str, config_from_dict, build_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_from_dict, build_spec)


def get_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise KeyError(f"unknown architecture {name!r}; known: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def known_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def register_part(role: str, kind: str, cls: type) -> None:
    if role not in PART_ROLES:
        raise KeyError(f"unknown part role {role!r}; known: {PART_ROLES}")
    _PARTS[(role, kind)] = cls


def get_part(role: str, kind: str) -> type:
    _ensure_builtin()
    if (role, kind) not in _PARTS:
        known = sorted(k for r, k in _PARTS if r == role)
        raise KeyError(f"unknown {role} kind {kind!r}; known: {known}")
    return _PARTS[(role, kind)]


def load_config(folder: str):
    """Read `folder/config.json`; return (architecture, typed configuration)."""
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path} not found: a model folder holds config.json and model.safetensors")
    with open(path) as f:
        raw = json.load(f)
    names = raw.get("architectures")
    if not names:
        raise KeyError(f"{path} has no 'architectures' entry; known architectures: {known_architectures()}")
    arch = get_architecture(names[0])
    return arch, arch.config_from_dict(raw)


_builtin_loaded = False


def _ensure_builtin() -> None:
    global _builtin_loaded
    if not _builtin_loaded:
        _builtin_loaded = True
        from . import parts  # noqa: F401  (registers the part kinds)
        from .models import llama  # noqa: F401  (registers LlamaForCausalLM)
