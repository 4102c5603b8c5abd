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
from .base import (BLOCKS, Block, DeferredBranch, FeedForward, Mixer, Norm, Part, ResidualStream, StepContext, branch_tensor,
                   forward_declares)


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    def __init__(self, mixer_norm: Norm, mixer: Mixer, ff_norm: Norm, feed_forward: FeedForward,
                 residual_scale: float = 1.0):
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ff_norm = ff_norm
        self.feed_forward = feed_forward
        self.residual_scale = float(residual_scale)
        # a part whose forward can leave its last product to the norm after it is asked to; the class that
        # defines ``forward`` says so itself, so a subclass with a forward of its own is asked only if it
        # declares the same
        self._mixer_defers = forward_declares(mixer, "can_defer_last")
        self._ff_defers = forward_declares(feed_forward, "can_defer_last")

    def parts(self) -> List[Part]:
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    @staticmethod
    def _normed(norm: Norm, deferred: bool, x, branch, branch_scale, ctx):
        """The normed rows and None, or (if the consumer finishes the norm itself) the rows without the norm's
        row factor and that factor's ingredients."""
        if not norm.takes_deferred_branch:
            branch = branch_tensor(branch)
        # a norm that takes a branch's last product over runs it in the same kernel: the label says so
        label = "norm+" + branch.tag.split(".")[-1] if isinstance(branch, DeferredBranch) else "norm"
        with ctx.timed(label):
            if deferred:
                hs = norm.forward_unscaled(x, branch, branch_scale, ctx, tag="block.h")
                if hs is not None:
                    return hs
            return norm.forward(x, branch, branch_scale, ctx, tag="block.h"), None

    def _mix(self, stream, ctx, cache, writes_cache):
        n = stream.x.shape[0]
        h, rs = self._normed(self.mixer_norm, self.mixer.takes_row_scale(n, ctx, cache, writes_cache),
                             stream.x, stream.take_pending(), stream.pending_scale, ctx)
        kw = {"defer_last": True} if self._mixer_defers else {}
        if rs is not None:
            kw["row_scale"] = rs
        return self.mixer.forward(h, ctx, cache, writes_cache, **kw)

    def _feed(self, stream, a, ctx):
        n = stream.x.shape[0]
        h, rs = self._normed(self.ff_norm, self.feed_forward.takes_row_scale(n, ctx),
                             stream.x, a, self.residual_scale, ctx)
        kw = {"defer_last": True} if self._ff_defers else {}
        if rs is not None:
            kw["row_scale"] = rs
        return self.feed_forward.forward(h, ctx, **kw)

    def forward(self, stream: ResidualStream, ctx: StepContext, cache: Optional[CacheView], writes_cache: bool = True):
        # the reference's timer labels distinguish prefill from decode and attention from feed-forward
        # (src/model/minicpm4/minicpm4_layer.cuh:46-83); the parts inside time their own kernels by class
        with ctx.timed("attn"):
            a = self._mix(stream, ctx, cache, writes_cache)
        with ctx.timed("ffn"):
            stream.pending = self._feed(stream, a, ctx)
        stream.pending_scale = self.residual_scale
