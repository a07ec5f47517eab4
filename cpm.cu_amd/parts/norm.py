"""RMSNorm with the residual add fused in front of it.

y = x * rsqrt(mean(x^2) + eps) * w  (src/model/norm.cuh:7-51); the branch of the
previous sub-layer is added into the residual stream by the same kernel
(src/model/norm.cuh:53-99), here with its scale and in float.
"""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .. import ops
from .base import (NORMS, BiasedBranch, DeferredBranch, Norm, NormedBranch, Runtime, StepContext, StreamsBranch, WeightSpec,
                   branch_tensor)


@NORMS.register("rms_norm")
class RMSNorm(Norm):
    """``unit_offset``: the checkpoint stores the weight around zero and the norm multiplies by 1 + w.
    ``scalar``: the checkpoint holds one number (a tensor without axes) that multiplies every coordinate."""

    def __init__(self, name: str, hidden_size: int, eps: float, unit_offset: bool = False, scalar: bool = False):
        self.name = name
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.unit_offset = bool(unit_offset)
        self.scalar = bool(scalar)

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.name, () if self.scalar else (self.hidden_size,),
                           "norm_offset" if self.unit_offset else "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        w = tensors[self.name].to(torch.float32)
        if self.scalar:
            w = w.reshape(1).expand(self.hidden_size)
        self.weight = (w + 1.0 if self.unit_offset else w).contiguous()
        self.rt = rt

    takes_deferred_branch = True
    takes_normed_branch = True

    def normalize(self, t, ctx: StepContext, tag="norm.plain"):
        if t.dim() == 3:                       # float partial sums of a split product
            t = t.sum(0) if t.shape[0] > 1 else t[0]
        out = ctx.ws.get(tag, (t.shape[0], self.hidden_size), torch.float32)
        ops.rms_norm_groups(t, self.weight, self.eps, out)
        return out

    def forward(self, x, branch, branch_scale, ctx: StepContext, rows=None, tag="norm"):
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = ctx.ws.get(tag, (n_out, self.hidden_size), self.rt.dtype)
        if isinstance(branch, NormedBranch) and isinstance(branch.norm, RMSNorm) and branch_scale == 1.0:
            # the branch's own norm, the residual add and this norm in one pass over the row
            ops.branch_norm_add_norm(x, branch_tensor(branch.branch), branch.norm.weight, branch.norm.eps,
                                     self.weight, self.eps, out, rows)
            return out
        branch = branch_tensor(branch)
        ops.add_rms_norm(x, branch, branch_scale, self.weight, self.eps, out, rows)
        return out

    def forward_streams(self, x, pending, read, ctx: StepContext, rows=None, tag="norm"):
        return _streams_norm(self, x, pending, read, ctx, rows, tag, rms=True)

    def forward_unscaled(self, x, branch, branch_scale, ctx: StepContext, tag="norm"):
        # decode steps: a row a workgroup leaves most of the chip idle, so the work is cut by columns and the
        # row factor rsqrt(mean(x^2) + eps) is left to the product that follows
        n = x.shape[0]
        if isinstance(branch, NormedBranch):
            return None
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


def _streams_norm(norm, x, pending: Optional[StreamsBranch], read, ctx: StepContext, rows, tag: str, rms: bool):
    n_out = x.shape[-2] if rows is None else rows.shape[0]
    out = ctx.ws.get(tag, (n_out, norm.hidden_size), norm.rt.dtype)
    branch = bias = mix = outw = None
    if pending is not None:
        (branch, bias), mix, outw = pending.pieces(), pending.mix, pending.out
    ops.streams_norm(x, branch, bias, 1.0, mix, outw, read, norm.weight, norm.eps, out, rows, rms=rms)
    return out


@NORMS.register("layer_norm")
class LayerNorm(Norm):
    """Layer norm with a weight and no bias: y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w, statistics in
    float, with the residual add fused in front of it like RMSNorm's; it also reads a residual of several streams."""

    def __init__(self, name: str, hidden_size: int, eps: float):
        self.name = name
        self.hidden_size = hidden_size
        self.eps = float(eps)

    def weight_specs(self) -> List[WeightSpec]:
        return [WeightSpec(self.name, (self.hidden_size,), "norm")]

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime):
        self.weight = tensors[self.name].to(torch.float32).contiguous()
        self.rt = rt

    takes_biased_branch = True

    def forward(self, x, branch, branch_scale, ctx: StepContext, rows=None, tag="norm"):
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = ctx.ws.get(tag, (n_out, self.hidden_size), self.rt.dtype)
        bias = None
        if isinstance(branch, BiasedBranch):
            branch, bias = branch.branch, branch.bias
            if branch_scale != 1.0:
                raise ValueError("layer_norm: a branch with a pending bias cannot be scaled")
        ops.streams_norm(x, branch_tensor(branch), bias, branch_scale, None, None, None, self.weight, self.eps, out, rows)
        return out

    def forward_streams(self, x, pending, read, ctx: StepContext, rows=None, tag="norm"):
        return _streams_norm(self, x, pending, read, ctx, rows, tag, rms=False)
