"""Weights from safetensors, by tensor name.

File discovery follows the reference (cpmcu/llm.py:139-166): exactly one
``*.safetensors.index.json`` (its ``weight_map`` names the shards), else exactly
one ``*.safetensors``.  Tensors are kept as stored: bfloat16 stays bfloat16, a
tensor stored in 32-bit floats stays so, float16 becomes bfloat16, integer
tables become int32.  What the file holds is compared with what the model's
parts ask for, and every difference (missing, unexpected, wrong shape) is
reported in one error; the reference reports unknown names only and loads
whatever else it finds (src/model/model.cuh:138-141).
"""
from __future__ import annotations

import glob
import json
import os
from typing import Callable, Dict, Iterable, List, Optional, Tuple

import torch

from ..parts.base import WeightSpec


class WeightError(ValueError):
    """The checkpoint does not hold what the model needs."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def checkpoint_files(model_dir: str) -> List[str]:
    idx = sorted(glob.glob(os.path.join(model_dir, "*.safetensors.index.json")))
    if len(idx) > 1:
        raise WeightError(f"several *.safetensors.index.json files in {model_dir}: {[os.path.basename(i) for i in idx]}")
    if len(idx) == 1:
        with open(idx[0], "r", encoding="utf-8") as f:
            shards = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_dir, s) for s in shards]
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    if len(files) > 1:
        raise WeightError(f"several *.safetensors files in {model_dir} and no index: {[os.path.basename(i) for i in files]}")
    if not files:
        raise WeightError(f"no *.safetensors (or *.safetensors.index.json) file in {model_dir}")
    return files


def stored_dtype(t: torch.dtype) -> torch.dtype:
    """The dtype a checkpoint tensor is kept in."""
    if t in (torch.bfloat16, torch.float16):
        return torch.bfloat16
    if t in (torch.float32, torch.float64):
        return torch.float32
    if t in (torch.int8, torch.uint8, torch.int16, torch.int32, torch.int64, torch.bool):
        return torch.int32
    raise WeightError(f"checkpoint tensor of unsupported dtype {t}")


def checkpoint_names(model_dir: str) -> List[str]:
    from safetensors import safe_open
    names: List[str] = []
    for path in checkpoint_files(model_dir):
        with safe_open(path, framework="pt", device="cpu") as f:
            names.extend(f.keys())
    return names


def _compare(specs: Iterable[WeightSpec], found: Dict[str, Tuple[int, ...]], where: str):
    want = {s.name: tuple(s.shape) for s in specs}
    missing = sorted(n for n in want if n not in found)
    unexpected = sorted(n for n in found if n not in want)
    wrong = sorted((n, found[n], want[n]) for n in want if n in found and tuple(found[n]) != want[n])
    if missing or unexpected or wrong:
        lines = [f"{where} does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " +
                         ", ".join(f"{n} is {list(a)}, expected {list(b)}" for n, a, b in wrong))
        raise WeightError("\n".join(lines), missing, unexpected, wrong)


def load_tensors(model_dir: str, specs: List[WeightSpec], device="cpu",
                 split_fused: Optional[Callable] = None, ignore: Optional[Callable] = None
                 ) -> Dict[str, torch.Tensor]:
    """name -> tensor on ``device`` for every spec; raises WeightError with the full list of differences."""
    from safetensors import safe_open
    files = checkpoint_files(model_dir)
    # pass 1: names and shapes only
    found: Dict[str, Tuple[int, ...]] = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                if ignore is not None and ignore(name):
                    continue
                shape = tuple(f.get_slice(name).get_shape())
                parts = split_fused(name, torch.empty(shape, device="meta")) if split_fused is not None else None
                for n, t in (parts if parts is not None else [(name, torch.empty(shape, device="meta"))]):
                    if n in found:
                        raise WeightError(f"{model_dir}: tensor '{n}' occurs twice in the checkpoint")
                    found[n] = tuple(t.shape)
    _compare(specs, found, model_dir)
    # pass 2: the data, one tensor at a time
    out: Dict[str, torch.Tensor] = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                if ignore is not None and ignore(name):
                    continue
                t = f.get_tensor(name)
                parts = split_fused(name, t) if split_fused is not None else None
                for n, p in (parts if parts is not None else [(name, t)]):
                    out[n] = p.to(stored_dtype(p.dtype)).contiguous().to(device)
    return out
