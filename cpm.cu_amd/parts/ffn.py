"""SiLU-gated feed-forward: down( silu(x Wg^T) * (x Wu^T) ).

gate and up are one stacked product, gate rows first (src/model/ffn.cuh:31-59,
77-84); silu(g) * u in float (src/model/activation.cuh:6-18).
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import FEED_FORWARDS, DeferredBranch, FeedForward, Part, StepContext
from .linear import Linear


@FEED_FORWARDS.register("gated_silu")
class GatedFFN(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int):
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = Linear([(prefix + "gate_proj.weight", intermediate_size),
                               (prefix + "up_proj.weight", intermediate_size)], hidden_size)
        self.down = Linear([(prefix + "down_proj.weight", hidden_size)], intermediate_size)

    def parts(self) -> List[Part]:
        return [self.gate_up, self.down]

    def takes_row_scale(self, n: int, ctx: StepContext) -> bool:
        return self.gate_up.gated_takes_row_scale(n)

    can_defer_last = True

    def forward(self, h: torch.Tensor, ctx: StepContext, row_scale=None, defer_last: bool = False):
        with ctx.timed("ffn_gate_up"):
            act = self.gate_up.forward_gated(h, ctx, "ffn.gate_up", row_scale=row_scale)
        if defer_last and self.down.defers(act):
            return DeferredBranch(self.down, act, ctx, "ffn.down")
        with ctx.timed("ffn_down"):
            return self.down.forward(act, ctx, "ffn.down", out_dtype=torch.float32, partials=True)
