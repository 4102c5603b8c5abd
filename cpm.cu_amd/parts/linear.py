"""Linear layer: y = alpha * x . W^T with W [out, in] as in the checkpoint.

Several checkpoint tensors may be stacked on the output axis into one weight
(q, k, v; gate, up), as the reference lays them out contiguously so that one
product serves them all (src/model/minicpm4/minicpm4_attn.cuh:48-55,
src/model/ffn.cuh:44-50).
"""
from __future__ import annotations

from typing import List, Mapping, Optional, Sequence, Tuple

import torch

from .. import ops
from .base import Part, Runtime, StepContext, WeightSpec


class Linear(Part):
    def __init__(self, names: Sequence[Tuple[str, int]], in_features: int, init: str = "matrix"):
        self.names = list(names)
        self.in_features = in_features
        self.out_features = sum(r for _, r in self.names)
        self.init = init
        self.weight: Optional[torch.Tensor] = None

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(n, (r, self.in_features), self.init) for n, r in self.names]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        ws = [tensors[n] for n, _ in self.names]
        w = ws[0] if len(ws) == 1 else torch.cat(ws, dim=0)
        self.weight = w.to(rt.dtype).contiguous()
        self.rt = rt
        # a second copy laid out for the decode product (bf16 engine; costs the weight's size again)
        self.tiled = ops.TiledWeight(self.weight) if (rt.dtype == torch.bfloat16 and rt.tiled_weights) else None

    def reserve_workspace(self, ws, rt: Runtime, max_step_tokens: int, max_slots: int):
        # An engine whose forward passes never carry more rows than the decode product takes reads the re-laid
        # copy only: the checkpoint's layout (what the library's many-row product and the 32-bit kernels read)
        # is let go, which halves what the weights hold.
        if self.tiled is not None and max_step_tokens <= ops.SKINNY_MAX_ROWS and self.in_features % 8 == 0:
            self.weight = None

    def forward(self, x: torch.Tensor, ctx: StepContext, tag: str, out_dtype: Optional[torch.dtype] = None,
                alpha: float = 1.0, rows: Optional[int] = None, partials: bool = False) -> torch.Tensor:
        """x [n, in] -> [n, out] (the first ``rows`` output features only, if given).  With ``partials`` the
        result may come as float32 partial sums [S, n, out] over slices of the input axis, for a consumer
        that adds them up (the norm and the position-encoding kernels do)."""
        if self.weight is not None:
            w = self.weight if rows is None else self.weight[:rows]
            wt = self.tiled if rows is None else None
        else:                                     # the re-laid copy alone: its first strips serve the first rows
            w, wt = None, (self.tiled if rows is None else self.tiled.first_rows(rows))
        n, N = x.shape[0], (self.out_features if rows is None else rows)
        if partials and ops.skinny_ok(x):
            S = ops.skinny_split(n, N, self.in_features)
            if S > 1:
                out = ctx.ws.get(tag, (S, n, N), torch.float32)
                ops.gemm_skinny(x, wt if wt is not None else w, out, alpha, mode="partial")
                return out
        out_dtype = out_dtype or x.dtype
        if partials and alpha == 1.0 and ops.library_gemm_ok(x, x.dtype):
            out_dtype = x.dtype         # many rows: the branch comes back in bf16 from the library product
        out = ctx.ws.get(tag, (n, N), out_dtype)
        ops.linear(x, w, out, alpha, w_tiled=wt)
        return out

    def defers(self, x: torch.Tensor) -> bool:
        """Whether, for these rows, a norm could run this product itself (ops.proj_add_norm): only then is it
        worth handing the product over instead of running it."""
        return (self.tiled is not None and x.dtype == torch.bfloat16 and ops.strip_kernels_ok(x.shape[0], self.in_features)
                and self.in_features % 8 == 0 and self.out_features % 4 == 0)

    def _gated_skinny(self, n: int, dtype) -> bool:
        return (dtype == torch.bfloat16 and n <= ops.SKINNY_MAX_ROWS and self.in_features % 8 == 0
                and (self.tiled is None or (self.out_features // 2) % 16 == 0))

    def gated_takes_row_scale(self, n: int) -> bool:
        """Whether forward_gated, for n rows, runs the kernel that can finish a norm (ops.RowScale)."""
        return self._gated_skinny(n, self.rt.dtype)

    def forward_gated(self, x: torch.Tensor, ctx: StepContext, tag: str, row_scale=None) -> torch.Tensor:
        """For a weight of gate rows stacked on up rows: silu(x Wg^T) * (x Wu^T), [n, out/2]."""
        n, half = x.shape[0], self.out_features // 2
        act = ctx.ws.get(tag + ".act", (n, half), x.dtype)
        if (n <= ops.STRIP_ROWS and x.dtype == torch.bfloat16 and self.tiled is not None and half % 16 == 0
                and self.in_features % 8 == 0):
            ops.gated_strip(x, self.tiled, act, row_scale=row_scale)      # a strip of columns a workgroup
        elif self._gated_skinny(n, x.dtype):
            ops.gemm_skinny(x, self.tiled if self.tiled is not None else self.weight, act, mode="gated",
                            row_scale=row_scale)
        else:
            if row_scale is not None:
                raise ValueError("forward_gated: a row scale needs the few-rows kernel (gated_takes_row_scale)")
            gu = self.forward(x, ctx, tag)
            ops.silu_mul(gu, act)
        return act
