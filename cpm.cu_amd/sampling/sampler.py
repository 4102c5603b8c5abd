"""Next-token choice: greedy, or a draw at a temperature.

The reference takes argmax when temperature is 0 and otherwise draws from
softmax(logits / temperature) with a seeded generator (cpmcu/llm.py:55-59,
282-285); it has no top-k, top-p or penalties, and neither has this sampler.
A draw is keyed by (seed, request id, number of tokens the request has
generated), so it does not depend on the rest of the batch.
"""
from __future__ import annotations

import os
from typing import Optional, Sequence

import torch

from .. import ops


class Sampler:
    def __init__(self, temperature: float = 0.0, seed: Optional[int] = None):
        if temperature < 0:
            raise ValueError(f"temperature {temperature} must be >= 0")
        self.temperature = float(temperature)
        # no seed given: draws differ from run to run, as an unseeded generator's would
        self.seed = int(seed) if seed is not None else int.from_bytes(os.urandom(8), "little")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0

    def sample(self, logits: torch.Tensor, request_ids: Sequence[int], steps: Sequence[int]) -> torch.Tensor:
        """int32 [rows]: one token per row of float32 logits [rows, vocab]."""
        rows = logits.shape[0]
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
        if self.greedy:
            ops.argmax(logits, out)
        else:
            meta = torch.tensor([list(request_ids), list(steps)], dtype=torch.int32).to(logits.device)
            ops.sample(logits, self.temperature, self.seed, meta[0].contiguous(), meta[1].contiguous(), out)
        return out
