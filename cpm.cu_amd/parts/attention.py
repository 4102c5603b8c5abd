"""Attention mixers: dense causal GQA attention, and InfLLM-v2 block-sparse
attention on top of it.

Dense (src/model/attn.cuh:58-284): q, k, v from one stacked product, position
encoding on q and k, k and v into the cache (the cache holds encoded keys),
attention of every query over its sequence's cached keys up to itself, output
projection.  scores = (q.k) * head_dim^-1/2; query head h reads kv head
h // (heads / kv_heads).

InfLLM-v2 (src/model/minicpm4/minicpm4_attn.cuh:107-202): past ``dense_len``
tokens a query attends only to chosen blocks of keys: blocks scored through
compressed keys (means of kernel_size keys every kernel_stride), the top-k of
them, plus initial blocks and a trailing window.  The reference selects per
call; here the selection of the query at position p uses only what lies before
p, so it does not depend on how the tokens were cut into steps:
compressed key j is visible iff kernel_stride*j + kernel_size <= p.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from ..cache.paged import CacheNeeds, CacheView, StreamSpec
from .base import MIXERS, DeferredBranch, Mixer, Part, PositionEncoding, Runtime, StepContext
from .linear import Linear


@MIXERS.register("gqa_attention")
class GQAAttention(Mixer):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], scale: Optional[float] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim <= 0 or head_dim % 16 or head_dim > 256:
            # the cache lays keys and values out in pieces of 16 features (the matrix cores' operands), and the
            # plain attention kernel holds a head in 256 features; said here so that no engine is built that
            # would fail at its first step
            raise ValueError(f"attention: head_dim {head_dim} is not supported: the cache and attention kernels take "
                             f"head sizes in steps of 16 up to 256")
        self.hidden_size = hidden_size
        self.nh, self.nkv, self.hd = num_heads, num_kv_heads, head_dim
        self.position = position
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.qkv = Linear([(prefix + "q_proj.weight", num_heads * head_dim),
                           (prefix + "k_proj.weight", num_kv_heads * head_dim),
                           (prefix + "v_proj.weight", num_kv_heads * head_dim)], hidden_size)
        self.o = Linear([(prefix + "o_proj.weight", hidden_size)], num_heads * head_dim)

    def parts(self) -> List[Part]:
        return [self.qkv, self.o] + ([self.position] if self.position is not None else [])

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.rt = rt
        self._qkv_fused = None               # the q/k/v weight re-laid for the fused decode kernel, made at first use

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        # the q/k/v weight in the fused decode kernel's order, if any step of this engine can run that kernel
        plain_rotation = self._kernel_rotates()
        if (self._qkv_fused is None and plain_rotation and rt.dtype == torch.bfloat16 and self.qkv.tiled is not None
                and self.hd % 16 == 0 and self.hidden_size % 8 == 0 and rt.page_size % 32 == 0):
            self._qkv_fused = ops.qkv_rope_weight(self.qkv.weight, self.nh, self.nkv, self.hd)
        # split-KV shares of steps of few tokens: their number grows with the context
        if rt.dtype == torch.bfloat16:
            most = max((n * ops.attention_splits(n, self.nkv, self.nh // self.nkv, rt.max_seq_len)
                        for n in range(1, min(max_step_tokens, ops.compute_units()) + 1)), default=0)
            if most > 1:
                ws.get("attn.part_o", (most, self.nh, self.hd), torch.float32)
                ws.get("attn.part_ml", (most, self.nh, 2), torch.float32)

    def cache_needs(self) -> CacheNeeds:
        w = self.nkv * self.hd
        return CacheNeeds(streams=(("k", StreamSpec(w)), ("v", StreamSpec(w))))

    def _kernel_rotates(self) -> bool:
        """Whether the projection kernels do all that the position encoding asks of q and k: a rotate-half
        rotation, or nothing (no encoding, or one that only biases the scores)."""
        return (self.position is None or self.position.rotary_params() is not None
                or not self.position.rewrites_vectors())

    # -- steps of forward, so that a subclass can put its own between them --
    def _fused_projection(self, n: int, dtype, cache: Optional[CacheView], writes_cache: bool) -> bool:
        """Decode steps: projection, rotation and cache write in one kernel (one kernel of the chain less)."""
        plain_rotation = self._kernel_rotates()
        return (writes_cache and cache is not None and plain_rotation and n <= ops.QKV_ROPE_MAX_ROWS
                and dtype == torch.bfloat16 and self.qkv.tiled is not None and self.hd % 16 == 0
                and self.hidden_size % 8 == 0 and cache.page_size % 32 == 0)

    def takes_row_scale(self, n: int, ctx: StepContext, cache, writes_cache: bool) -> bool:
        return self._fused_projection(n, self.rt.dtype, cache, writes_cache)

    def project_and_store(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool, row_scale=None,
                          compress=None) -> torch.Tensor:
        """q [n, heads * head_dim], position-encoded; k and v go into the cache.  ``compress`` (a pool of
        compressed keys, kernel_size, kernel_stride) is only given where _fused_projection() holds: that kernel
        then also writes the compressed keys that the step's tokens complete."""
        n = h.shape[0]
        nh, nkv, hd = self.nh, self.nkv, self.hd
        plain_rotation = self._kernel_rotates()
        if self._fused_projection(n, h.dtype, cache, writes_cache):
            if self._qkv_fused is None:           # a part used outside an engine (reserve_workspace makes it)
                self._qkv_fused = ops.qkv_rope_weight(self.qkv.weight, nh, nkv, hd)
            rot = self.position.rotary_params() if self.position is not None else None
            inv_freq, mag = (rot if rot is not None else (None, 1.0))
            q = ctx.ws.get("attn.q", (n, nh * hd), self.rt.dtype)
            ops.qkv_rope(h, self._qkv_fused, q, nh, nkv, hd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                         cache.streams["k"], cache.streams["v"], cache.page_table, cache.page_size,
                         row_scale=row_scale, compress=compress)
            return q
        if row_scale is not None or compress is not None:
            raise ValueError("attention: a row scale or compressed keys need the fused projection (takes_row_scale)")
        qkv = self.qkv.forward(h, ctx, "attn.qkv", rows=None if writes_cache else nh * hd, partials=plain_rotation)
        rot = self.position.rotary_params() if self.position is not None else None
        inv_freq, mag = (rot if rot is not None else (None, 1.0))
        if self.position is not None and rot is None and self.position.rewrites_vectors():
            q3 = qkv[:, :nh * hd].unflatten(1, (nh, hd))
            k3 = qkv[:, nh * hd:(nh + nkv) * hd].unflatten(1, (nkv, hd)) if writes_cache else None
            self.position.apply(q3, k3, ctx)
        q = ctx.ws.get("attn.q", (n, nh * hd), self.rt.dtype)
        ops.rope_store(qkv, q, nh, nkv, hd, ctx.positions, ctx.tok_slot, inv_freq, mag,
                       cache.streams["k"] if writes_cache else None, cache.streams["v"] if writes_cache else None,
                       cache.page_table if writes_cache else None, cache.page_size, writes_cache)
        return q

    can_defer_last = True

    def attend_and_project(self, q, ctx: StepContext, cache: CacheView, sel=None, defer_last: bool = False):
        """Attention of q over the cache (all keys up to each query, or the blocks listed in ``sel``), then the
        output projection."""
        sel_blocks, sel_count, bs, window_blocks = sel if sel is not None else (None, None, 0, 0)
        out = ctx.ws.get("attn.out", tuple(q.shape), q.dtype)
        slopes = self.position.score_bias() if self.position is not None else None
        with ctx.timed("attn_core"):
            ops.attention(q, out, self.nh, self.nkv, self.hd, self.scale, cache.streams["k"], cache.streams["v"],
                          cache.page_table, cache.page_size, ctx, sel_blocks, sel_count, bs, window_blocks,
                          head_slopes=slopes)
        if defer_last and self.o.defers(out):
            return DeferredBranch(self.o, out, ctx, "attn.o")
        with ctx.timed("attn_o"):
            return self.o.forward(out, ctx, "attn.o", out_dtype=torch.float32, partials=True)

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True, row_scale=None,
                defer_last: bool = False):
        with ctx.timed("attn_qkv_rope"):
            q = self.project_and_store(h, ctx, cache, writes_cache, row_scale)
        return self.attend_and_project(q, ctx, cache, defer_last=defer_last)


@MIXERS.register("infllm_v2_attention")
class InfLLMv2Attention(GQAAttention):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: Optional[PositionEncoding], kernel_size: int, kernel_stride: int, block_size: int,
                 init_blocks: int, topk: int, window_size: int, dense_len: int, scale: Optional[float] = None):
        super().__init__(prefix, hidden_size, num_heads, num_kv_heads, head_dim, position, scale)
        if block_size % kernel_stride or kernel_size < kernel_stride:
            raise ValueError("infllm_v2: block_size must be a multiple of kernel_stride <= kernel_size")
        if window_size % block_size or window_size < block_size:
            raise ValueError("infllm_v2: window_size must be a positive multiple of block_size")
        self.ks, self.st, self.bs = kernel_size, kernel_stride, block_size
        self.init_blocks, self.topk, self.dense_len = init_blocks, topk, dense_len
        self.window_blocks = window_size // block_size

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        super().bind(tensors, rt)
        if rt.page_size % self.st:
            raise ValueError(f"infllm_v2: kernel_stride {self.st} must divide the cache page of {rt.page_size} tokens "
                             f"(a compressed key's row lies in the page of its first key)")

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        super().reserve_workspace(ws, rt, max_step_tokens, max_slots)
        # the selection's scores grow with the context: sized here for the longest sequence, for steps of few
        # tokens (many small workgroups through scratch) and of many
        few = max(256 // self.nkv, 1)
        need = max(ops.sparse_select_scratch(rt.dtype, n, self.nh, self.nkv, self.hd, rt.max_seq_len - 1, self.ks,
                                             self.st, self.bs)
                   for n in {1, min(few, max_step_tokens), min(few + 1, max_step_tokens), max_step_tokens})
        if need:
            ws.get("attn.sel_scores", (need,), torch.float32)
        # the block lists of the largest step (a rehearsal pass at short positions never selects)
        ws.get("attn.sel_blocks", (max_step_tokens, self.nkv, self.topk + self.window_blocks), torch.int32)
        ws.get("attn.sel_count", (max_step_tokens, self.nkv), torch.int32)

    def cache_needs(self) -> CacheNeeds:
        w = self.nkv * self.hd
        return CacheNeeds(streams=(("k", StreamSpec(w)), ("v", StreamSpec(w)), ("ck", StreamSpec(w, every=self.st))))

    can_defer_last = True

    def forward(self, h, ctx: StepContext, cache: CacheView, writes_cache: bool = True, row_scale=None,
                defer_last: bool = False):
        # decode steps: the projection kernel completes the compressed keys itself (one kernel of the chain less)
        fused = self._fused_projection(h.shape[0], h.dtype, cache, writes_cache)
        with ctx.timed("attn_qkv_rope"):
            q = self.project_and_store(h, ctx, cache, writes_cache, row_scale,
                                       compress=(cache.streams["ck"], self.ks, self.st) if fused else None)
        if writes_cache and not fused:
            with ctx.timed("attn_compress"):
                ops.compress_keys(cache.streams["k"], cache.streams["ck"], self.nkv, cache.page_table,
                                  cache.page_size, ctx.positions, ctx.tok_slot, self.ks, self.st)
        sel = None
        if ctx.max_pos + 1 > self.dense_len:
            n = q.shape[0]
            max_sel = self.topk + self.window_blocks
            sel_blocks = ctx.ws.get("attn.sel_blocks", (n, self.nkv, max_sel), torch.int32)
            sel_count = ctx.ws.get("attn.sel_count", (n, self.nkv), torch.int32)
            need = ops.sparse_select_scratch(q.dtype, n, self.nh, self.nkv, self.hd, ctx.max_pos, self.ks, self.st, self.bs)
            scratch = ctx.ws.get("attn.sel_scores", (need,), torch.float32) if need else None
            # the reference times its two selection stages apart (minicpm4_attn.cuh:107-202); here they are one call
            with ctx.timed("attn_select"):
                ops.sparse_select(q, cache.streams["ck"], self.nh, self.nkv, self.hd, self.scale, cache.page_table,
                                  cache.page_size, ctx.positions, ctx.tok_slot, self.ks, self.st, self.bs,
                                  self.init_blocks, self.topk, self.window_blocks, self.dense_len, ctx.max_pos,
                                  sel_blocks, sel_count, scratch=scratch)
            sel = (sel_blocks, sel_count, self.bs, self.window_blocks)
        return self.attend_and_project(q, ctx, cache, sel, defer_last=defer_last)
