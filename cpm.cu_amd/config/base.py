"""Typed configuration: the shared machinery.

A model configuration is a frozen dataclass whose fields are the keys of the
architecture's own config.json.  ``field_from`` reads one key with a type check
and says which key was wrong; nothing here knows any architecture.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional


class ConfigError(ValueError):
    """A config.json key is missing, of the wrong type, or inconsistent."""


_MISSING = object()


def field_from(raw: Dict[str, Any], key: str, kind: Callable, default: Any = _MISSING, where: str = "config.json"):
    """raw[key] converted with ``kind`` (int, float, bool, str); ``default`` if absent or null."""
    v = raw.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(f"{where}: required key '{key}' is missing")
        return default
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: '{key}' must be true or false, got {v!r}")
        return v
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                return int(v)
            raise ConfigError(f"{where}: '{key}' must be an integer, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: '{key}' must be a number, got {v!r}")
        return float(v)
    if kind is str:
        if not isinstance(v, str):
            raise ConfigError(f"{where}: '{key}' must be a string, got {v!r}")
        return v
    return kind(v)


def require(cond: bool, message: str):
    if not cond:
        raise ConfigError(message)


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir}")
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def architecture_name(raw: Dict[str, Any]) -> str:
    """The name the registry is keyed on: config.json's architectures[0]
    (the reference detects the family from the same key, cpmcu/common/utils.py:41-42)."""
    arch = raw.get("architectures")
    if not isinstance(arch, list) or not arch or not isinstance(arch[0], str):
        raise ConfigError("config.json: 'architectures' must be a non-empty list of names")
    return arch[0]


@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration."""
    architecture: str

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":  # pragma: no cover - interface
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:  # pragma: no cover - interface
        """config.json content that from_dict reads back to an equal object."""
        raise NotImplementedError

    # What the engine, the generation loop and the front end ask of any configuration, whatever its own
    # keys are called:
    @property
    def stop_token_ids(self):
        """Token ids that end a sequence."""
        return ()

    @property
    def vocabulary_size(self) -> int:  # pragma: no cover - interface
        raise NotImplementedError

    @property
    def longest_sequence(self) -> Optional[int]:
        """Positions the model is meant for (None: no limit of its own); the engine's default max_seq_len."""
        return None
