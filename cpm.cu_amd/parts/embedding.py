"""Token embedding (times its scale) and the output head.

x[t] = E[id_t] * scale_emb (src/model/embedding.cuh:7-20, 49-52); logits =
(y * head_scale) . W^T with the head reading the unscaled table when the
embeddings are tied (src/model/linear.cuh:86-105, cpmcu/llm.py:136-137).
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from .base import Part, Runtime, StepContext, WeightSpec


class TokenEmbedding(Part):
    def __init__(self, name: str, vocab_size: int, hidden_size: int, scale: float = 1.0):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.table: Optional[torch.Tensor] = None

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.name, (self.vocab_size, self.hidden_size), "table")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.table = tensors[self.name].to(rt.dtype).contiguous()

    def forward(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.ws.get("residual", (ctx.n_tokens, self.hidden_size), torch.float32)
        ops.embed(self.table, ctx.token_ids, x, self.scale)
        return x


class LMHead(Part):
    def __init__(self, name: str, vocab_size: int, hidden_size: int, scale: float = 1.0,
                 tied_to: Optional[TokenEmbedding] = None):
        self.name = name
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.scale = float(scale)
        self.tied_to = tied_to
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self) -> List[WeightSpec]:
        return [] if self.tied_to is not None else [WeightSpec(self.name, (self.vocab_size, self.hidden_size), "table")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        if self.tied_to is None:
            self.weight = tensors[self.name].to(rt.dtype).contiguous()
        self.rt = rt
        self.tiled = None

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        # the table in the decode product's layout (made here and not at bind: a tied table is bound by its owner)
        if self.tiled is None and rt.dtype == torch.bfloat16 and rt.tiled_weights:
            self.tiled = ops.TiledWeight(self.tied_to.table if self.tied_to is not None else self.weight)
        # logits are float32: every product of the head goes through the re-laid copy, whatever the number of rows,
        # so a head of its own lets the checkpoint's layout go (a tied head's table stays: the embedding reads it)
        if self.tiled is not None and self.tied_to is None and self.hidden_size % 8 == 0:
            self.weight = None

    def forward(self, y: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        w = self.tied_to.table if self.tied_to is not None else self.weight
        if self.tiled is None and self.rt.dtype == torch.bfloat16 and self.rt.tiled_weights:
            self.tiled = ops.TiledWeight(w)
        logits = ctx.ws.get("logits", (y.shape[0], self.vocab_size), torch.float32)
        ops.linear(y, w, logits, self.scale, w_tiled=self.tiled)
        return logits
