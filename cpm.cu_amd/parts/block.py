"""Arrangement of a layer's parts around the residual stream.

Pre-norm with scaled residual branches: x += s * Mixer(norm1(x)); x += s *
FeedForward(norm2(x)).  As in the reference each branch is added by the norm
that follows it (src/model/minicpm4/minicpm4_layer.cuh:42-62), so a block
leaves its feed-forward branch pending for the next block's first norm (or the
model's final norm).
"""
from __future__ import annotations

from typing import List, Optional

from ..cache.paged import CacheView
from .base import BLOCKS, Block, FeedForward, Mixer, Norm, Part, ResidualStream, StepContext


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ff_norm: Norm, feed_forward: FeedForward,
                 residual_scale: float = 1.0):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ff_norm = ff_norm
        self.feed_forward = feed_forward
        self.residual_scale = float(residual_scale)

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        if ctx.perf is not None and ctx.perf.enabled:
            # the reference's timer labels distinguish prefill from decode and attention from feed-forward
            # (src/model/minicpm4/minicpm4_layer.cuh:46-83)
            phase = "decode" if ctx.single_token else "prefill"
            with ctx.perf.gpu(f"{phase}_attn"):
                h = self.mixer_norm.forward(stream.x, stream.pending, stream.pending_scale, ctx, tag="block.h")
                a = self.mixer.forward(h, ctx, cache, writes_cache)
            with ctx.perf.gpu(f"{phase}_ffn"):
                h = self.ff_norm.forward(stream.x, a, self.residual_scale, ctx, tag="block.h")
                stream.pending = self.feed_forward.forward(h, ctx)
            stream.pending_scale = self.residual_scale
            return
        h = self.mixer_norm.forward(stream.x, stream.pending, stream.pending_scale, ctx, tag="block.h")
        a = self.mixer.forward(h, ctx, cache, writes_cache)
        h = self.ff_norm.forward(stream.x, a, self.residual_scale, ctx, tag="block.h")
        stream.pending = self.feed_forward.forward(h, ctx)
        stream.pending_scale = self.residual_scale
