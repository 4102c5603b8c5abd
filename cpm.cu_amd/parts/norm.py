"""RMSNorm with the residual add fused in front of it.

y = x * rsqrt(mean(x^2) + eps) * w  (src/model/norm.cuh:7-51); the branch of the
previous sub-layer is added into the residual stream by the same kernel
(src/model/norm.cuh:53-99), here with its scale and in float.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from .base import NORMS, DeferredBranch, Norm, Runtime, StepContext, WeightSpec, branch_tensor


@NORMS.register("rms_norm")
class RMSNorm(Norm):
    def __init__(self, name: str, hidden_size: int, eps: float):
        self.name = name
        self.hidden_size = hidden_size
        self.eps = float(eps)

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.name, (self.hidden_size,), "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.weight = tensors[self.name].to(torch.float32).contiguous()
        self.rt = rt

    takes_deferred_branch = True

    def forward(self, x, branch, branch_scale, ctx: StepContext, rows=None, tag="norm"):
        branch = branch_tensor(branch)
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = ctx.ws.get(tag, (n_out, self.hidden_size), self.rt.dtype)
        ops.add_rms_norm(x, branch, branch_scale, self.weight, self.eps, out, rows)
        return out

    def forward_unscaled(self, x, branch, branch_scale, ctx: StepContext, tag="norm"):
        # decode steps: a row a workgroup leaves most of the chip idle, so the work is cut by columns and the
        # row factor rsqrt(mean(x^2) + eps) is left to the product that follows
        n = x.shape[0]
        if self.rt.dtype != torch.bfloat16 or not ops.strip_kernels_ok(n, self.hidden_size) or self.hidden_size % 4:
            return None
        out = ctx.ws.get(tag, (n, self.hidden_size), torch.bfloat16)
        if isinstance(branch, DeferredBranch):
            # the branch's last product, the residual add and this norm's column work in one kernel: a workgroup
            # of that product owns 16 columns over all of K and finishes them itself
            lin = branch.linear
            fits = lin.out_features == self.hidden_size
            if fits and lin.defers(branch.a):
                sums = ctx.ws.get(tag + ".sums16", (n, -(-self.hidden_size // 16)), torch.float32)
                ops.proj_add_norm(branch.a, lin.tiled, branch_scale, x, self.weight, out, sums)
                return out, ops.RowScale(sums, self.eps)
            branch = branch.evaluate()
        sums = ctx.ws.get(tag + ".sums", (n, ops.norm_slices(self.hidden_size)), torch.float32)
        ops.add_norm_columns(x, branch, branch_scale, self.weight, out, sums)
        return out, ops.RowScale(sums, self.eps)
