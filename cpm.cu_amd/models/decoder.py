"""A decoder-only model as data: parts, and the order in which they run.

``layers`` are blocks built from parts; ``schedule`` is the list of runs, each
naming the layer to run and the cache entry it uses.  A layer may be named by
several runs (its weights are shared; each run has a cache entry of its own
unless it says otherwise), and a run may read the cache entry that an earlier
run wrote instead of writing one (``writes_cache`` false): then the mixer only
projects queries.  The model itself knows nothing about what the parts compute.

Forward of a step (reference order: src/model/minicpm4/minicpm4_model.cuh:125-153):
embedding -> runs of the schedule -> final norm on the wanted rows -> head.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch

from ..cache.paged import CacheNeeds
from ..parts.base import Block, Norm, Part, ResidualStream, Runtime, StepContext
from ..parts.embedding import LMHead, TokenEmbedding


@dataclass(frozen=True)
class Run:
    layer: int                    # index into DecoderModel.layers
    cache: int                    # cache entry this run uses
    writes_cache: bool = True     # False: read the entry another run wrote


def sequential_schedule(n_layers: int) -> List[Run]:
    return [Run(i, i, True) for i in range(n_layers)]


class DecoderModel(Part):
    def __init__(self, config, embedding: TokenEmbedding, layers: Sequence[Block], final_norm: Norm, head: LMHead,
                 schedule: Optional[Sequence[Run]] = None):
        self.config = config
        self.embedding = embedding
        self.layers = list(layers)
        self.final_norm = final_norm
        self.head = head
        self.schedule = list(schedule) if schedule is not None else sequential_schedule(len(self.layers))
        self._check_schedule()

    def _check_schedule(self):
        written = set()
        for r in self.schedule:
            if not 0 <= r.layer < len(self.layers):
                raise ValueError(f"schedule names layer {r.layer}, the model has {len(self.layers)}")
            if r.writes_cache:
                if r.cache in written:
                    raise ValueError(f"cache entry {r.cache} is written by two runs of the schedule")
                written.add(r.cache)
            elif r.cache not in written:
                raise ValueError(f"a run reads cache entry {r.cache} before any run has written it")
        self.n_cache_entries = (max(written) + 1) if written else 0
        if written != set(range(self.n_cache_entries)):
            raise ValueError("cache entries of the schedule must be numbered 0..n-1 without gaps")

    @property
    def vocab_size(self) -> int:
        return self.head.vocab_size

    def parts(self) -> List[Part]:
        return [self.embedding] + self.layers + [self.final_norm, self.head]

    def cache_needs(self) -> List[CacheNeeds]:
        """What each cache entry needs: that of the mixer of the run that writes it."""
        needs: List[Optional[CacheNeeds]] = [None] * self.n_cache_entries
        for r in self.schedule:
            if r.writes_cache:
                needs[r.cache] = self.layers[r.layer].mixer.cache_needs()
        return needs  # type: ignore[return-value]

    def forward(self, ctx: StepContext) -> torch.Tensor:
        """float32 logits [R, V] at ctx.logit_rows; the step's tokens enter the cache."""
        with ctx.timed("embed"):
            stream = ResidualStream(self.embedding.forward(ctx))
        for r in self.schedule:
            self.layers[r.layer].forward(stream, ctx, ctx.cache.view(r.cache) if ctx.cache is not None else None,
                                         r.writes_cache)
        if ctx.logit_rows is None or ctx.logit_rows.numel() == 0:
            return None
        with ctx.timed("head"):
            y = self.final_norm.forward(stream.x, stream.pending, stream.pending_scale, ctx, rows=ctx.logit_rows,
                                        tag="final.y")
            return self.head.forward(y, ctx)
