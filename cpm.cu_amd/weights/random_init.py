"""Random weights: a model folder (config.json, model.safetensors) from a configuration and a seed.

The reference has no such mode.  Every tensor is drawn from a generator keyed by
(seed, tensor name), so a tensor's values depend on nothing but those two and
its shape: matrices and tables N(0, std), norm weights 1 + N(0, norm_std).
Values are stored in bfloat16 (the checkpoint's dtype), or as each spec says.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Callable, Dict, Optional

import torch

from ..config.base import ModelConfig
from ..parts.base import WeightSpec
from ..registry import get_architecture

_STORAGE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "int32": torch.int32}


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF)
    return g


# init rule name (WeightSpec.init) -> function(spec, generator, device, dtype, std, norm_std) -> tensor of
# spec.shape in dtype.  A part with another kind of tensor (decay rates, convolution taps) registers its own
# rule under a new name and names it in its WeightSpecs; this file needs no change for it.
INIT_RULES: Dict[str, Callable] = {}


def register_init_rule(name: str, fn: Optional[Callable] = None):
    def deco(f):
        if name in INIT_RULES and INIT_RULES[name] is not f:
            raise ValueError(f"init rule '{name}' is already registered")
        INIT_RULES[name] = f
        return f
    return deco if fn is None else deco(fn)


@register_init_rule("norm")
def _init_norm(spec, g, device, dtype, std, norm_std):
    """1 + N(0, norm_std)."""
    t = torch.ones(spec.shape, dtype=torch.float32, device=device)
    if norm_std > 0:
        t += torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * norm_std
    return t.to(dtype)


@register_init_rule("matrix")
def _init_matrix(spec, g, device, dtype, std, norm_std):
    """N(0, std)."""
    if len(spec.shape) == 2 and spec.shape[0] * spec.shape[1] > (1 << 28):
        # large tables row-block by row-block, to bound the float32 temporary
        out = torch.empty(spec.shape, dtype=dtype, device=device)
        step = max((1 << 28) // spec.shape[1], 1)
        for r in range(0, spec.shape[0], step):
            rows = min(step, spec.shape[0] - r)
            out[r:r + rows] = (torch.randn((rows, spec.shape[1]), generator=g, dtype=torch.float32, device=device)
                               * std).to(dtype)
        return out
    return (torch.randn(spec.shape, generator=g, dtype=torch.float32, device=device) * std).to(dtype)


register_init_rule("table", _init_matrix)


def draw(spec: WeightSpec, seed: int, std: float = 0.02, norm_std: float = 0.0, device="cpu") -> torch.Tensor:
    g = _generator(seed, spec.name, device)
    rule = INIT_RULES.get(spec.init)
    if rule is None:
        raise ValueError(f"tensor '{spec.name}': unknown init rule '{spec.init}' (registered: {sorted(INIT_RULES)})")
    t = rule(spec, g, device, _STORAGE[spec.storage], std, norm_std)
    if tuple(t.shape) != tuple(spec.shape) or t.dtype != _STORAGE[spec.storage]:
        raise ValueError(f"tensor '{spec.name}': init rule '{spec.init}' gave {tuple(t.shape)} {t.dtype}, "
                         f"{tuple(spec.shape)} {_STORAGE[spec.storage]} expected")
    return t


def random_tensors(config: ModelConfig, seed: int, std: float = 0.02, norm_std: float = 0.0, device="cpu"
                   ) -> Dict[str, torch.Tensor]:
    """All tensors the architecture's model asks for, drawn from (seed, name)."""
    model = get_architecture(config.architecture).build_model(config)
    return {s.name: draw(s, seed, std, norm_std, device) for s in model.all_weight_specs()}


def write_model_dir(config: ModelConfig, out_dir: str, seed: int, std: float = 0.02, norm_std: float = 0.0) -> str:
    """Write config.json and model.safetensors for ``config`` into out_dir."""
    from safetensors.torch import save_file
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config.to_dict(), f, indent=2)
    tensors = random_tensors(config, seed, std, norm_std)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    return out_dir
