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
        self._meta: Optional[torch.Tensor] = None

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
            meta = self._upload(logits.device, request_ids, steps)
            ops.sample(logits, self.temperature, self.seed, meta[0, :rows], meta[1, :rows], out)
        return out

    def _upload(self, device, request_ids: Sequence[int], steps: Sequence[int]) -> torch.Tensor:
        """Request ids and step numbers on the device, int32 [2, rows]: through a pinned buffer and into a device
        buffer that both live as long as the sampler, so that a decode loop allocates nothing for them."""
        rows = len(request_ids)
        if self._meta is None or self._meta.shape[1] < rows or self._meta.device != device:
            cap = max(rows, 64)
            self._meta = torch.empty((2, cap), dtype=torch.int32, device=device)
            self._stage = [torch.empty((2, cap), dtype=torch.int32).pin_memory() if device.type == "cuda"
                           else torch.empty((2, cap), dtype=torch.int32) for _ in range(2)]
            self._events = [None, None]
            self._turn = 0
        i = self._turn
        self._turn ^= 1
        if self._events[i] is not None:
            self._events[i].synchronize()            # the copy that last used this staging buffer has finished
        st = self._stage[i]
        st[0, :rows] = torch.as_tensor(list(request_ids), dtype=torch.int32)
        st[1, :rows] = torch.as_tensor(list(steps), dtype=torch.int32)
        self._meta[:, :rows].copy_(st[:, :rows], non_blocking=True)
        if device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self._events[i] = ev
        return self._meta
