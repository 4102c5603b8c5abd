"""One registry from an architecture's name (config.json ``architectures[0]``) to its model.

An architecture brings: its typed configuration class, a function that builds the
model (parts and schedule) from a configuration, and the checkpoint's
peculiarities (fused tensors to split, tensors to ignore).  The reference
chooses the model class from the same config key (cpmcu/common/utils.py:33-64).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional


@dataclass
class Architecture:
    name: str
    config_class: type
    build: Callable                                  # (config, tied=None) -> model
    split_fused: Optional[Callable] = None           # (config, name, tensor) -> [(name, tensor)] or None
    ignore_tensor: Optional[Callable] = None         # (config, name) -> bool
    tie_key: Optional[str] = None                    # tensor whose absence means tied embeddings when config is silent


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False):
    if arch.name in _ARCHITECTURES and not replace and _ARCHITECTURES[arch.name] is not arch:
        raise ValueError(f"architecture '{arch.name}' is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str):
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise KeyError(f"unknown architecture '{name}' (registered: {sorted(_ARCHITECTURES)})") from None


def architectures() -> List[str]:
    return sorted(_ARCHITECTURES)
