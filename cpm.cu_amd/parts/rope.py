"""Rotary position encoding, plain and LongRoPE.

Rotate-half rotation by theta = position * inv_freq[c] (src/model/rotary.cuh:7-34).
The reference loads inv_freq once, computed for the engine's whole token budget
(cpmcu/llm.py:181-191): the choice between LongRoPE's short and long factors is
static per engine, long iff the engine holds sequences longer than
original_max_position_embeddings.  inv_freq[c] = 1 / (factor[c] * theta^(2c/hd)).
cos and sin carry the magnitude m = sqrt(1 + ln(max_position/original_max) /
ln(original_max)) when the position range was stretched (the reference drops it,
cpmcu/llm.py:190-192; ``attention_scaling=False`` does the same).
"""
from __future__ import annotations

import math
from typing import Mapping, Optional, Sequence, Tuple

import torch

from .base import POSITION_ENCODINGS, PositionEncoding, Runtime


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    def __init__(self, head_dim: int, theta: float):
        self.head_dim = head_dim
        self.theta = float(theta)
        self.inv_freq: Optional[torch.Tensor] = None
        self.magnitude = 1.0

    def factors(self, max_seq_len: int) -> Optional[Sequence[float]]:
        return None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        c = torch.arange(0, self.head_dim, 2, dtype=torch.float64)
        base = self.theta ** (c / self.head_dim)
        f = self.factors(rt.max_seq_len)
        if f is not None:
            base = base * torch.tensor(list(f), dtype=torch.float64)
        self.inv_freq = (1.0 / base).to(torch.float32).to(rt.device)

    def rotary_params(self) -> Tuple[torch.Tensor, float]:
        return self.inv_freq, self.magnitude


@POSITION_ENCODINGS.register("longrope")
class LongRotaryEncoding(RotaryEncoding):
    def __init__(self, head_dim: int, theta: float, short_factor: Sequence[float], long_factor: Sequence[float],
                 original_max_position: int, max_position: int, attention_scaling: bool = True):
        super().__init__(head_dim, theta)
        if len(short_factor) != head_dim // 2 or len(long_factor) != head_dim // 2:
            raise ValueError(f"longrope: factor lists need head_dim/2 = {head_dim // 2} entries")
        self.short_factor = tuple(short_factor)
        self.long_factor = tuple(long_factor)
        self.original_max_position = original_max_position
        self.max_position = max_position
        ratio = max_position / original_max_position
        if attention_scaling and ratio > 1.0:
            self.magnitude = math.sqrt(1.0 + math.log(ratio) / math.log(original_max_position))

    def factors(self, max_seq_len: int):
        return self.long_factor if max_seq_len > self.original_max_position else self.short_factor
