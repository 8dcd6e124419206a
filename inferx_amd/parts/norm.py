"""RMSNorm, fused with the residual add that precedes it.

y = v * rsqrt(mean(v^2) + eps) * weight with v = h + delta, everything in
float32, rounded once (reference: RmsNormKernel, src/backends/cuda/ops/layers.cu:50-76).
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import LazyDelta, Norm, ParamSpec, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, width: int, eps: float, scalar: bool = False, groups: int = 1):
        """`scalar`: the weight is ONE number for all coordinates (a tensor without dimensions), spread over the
        width when it is bound, so that every kernel that applies an RMS norm takes it as it is.  `groups`: the
        width is cut into that many equal consecutive runs, and each is divided by its own root mean square."""
        self.width, self.eps, self.scalar, self.groups = int(width), float(eps), bool(scalar), int(groups)
        if self.groups < 1 or self.width % self.groups:
            raise ValueError(f"{groups} groups do not divide a width of {width}")
        self.weight = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", () if self.scalar else (self.width,), init="ones")]

    def bind(self, tensors, rt) -> None:
        w = tensors["weight"]
        self.weight = w.reshape(1).expand(self.width).contiguous() if self.scalar else w.contiguous()

    def rms_operands(self):
        # (a norm in groups is not the plain one that other kernels know how to apply on their way)
        return (self.weight, self.eps) if self.groups == 1 else None

    def forward(self, ctx, h, delta=None, rows=None):
        """h [T, width] float32 is updated in place with `delta` (unless `rows`
        picks rows out); returns the normalised rows in the run's type."""
        n = h.shape[0] if rows is None else rows.numel()
        out = ctx.rt.empty((n, self.width))
        if isinstance(delta, LazyDelta):
            if self.groups == 1:
                if delta.add_rmsnorm(ctx, h, self.weight, self.eps, rows, out):
                    return out
            elif getattr(delta, "norms_in_groups", False):  # a sum that knows how to ride on a norm in groups
                if delta.add_rmsnorm(ctx, h, self.weight, self.eps, rows, out, groups=self.groups):
                    return out
            delta = delta.materialize(ctx)
        ops.add_rmsnorm(h, delta, self.weight, out, self.eps, rows, self.groups)
        return out


class NormedDelta(LazyDelta):
    """A branch's result that passes a norm of its own before it is added to the residual stream (layers with a
    norm before and after each branch): norm(delta), not formed yet.  `delta` may itself be a sum that is not formed
    yet.  An RMS norm that consumes it forms it, adds it and normalises the sum in one kernel; anybody else gets the
    normalised tensor in float32."""

    def __init__(self, delta, norm: Norm):
        self.delta, self.norm = delta, norm

    def tensor(self, ctx):
        if isinstance(self.delta, LazyDelta):
            self.delta = self.delta.materialize(ctx)
        return self.delta

    def materialize(self, ctx):
        tensor = self.tensor(ctx)
        zeros = torch.zeros(tuple(tensor.shape), dtype=torch.float32, device=tensor.device)
        rms = self.norm.rms_operands()
        if rms is None:  # some other norm: through its own forward, in the run's type
            return self.norm.forward(ctx, zeros, tensor)
        out = torch.empty_like(zeros)
        ops.add_rmsnorm(zeros, tensor, rms[0], out, rms[1])
        return out

    def add_rmsnorm(self, ctx, h, weight, eps, rows, out) -> bool:
        rms = self.norm.rms_operands()
        if rms is None:
            return False
        fused = getattr(self.delta, "add_normed_rmsnorm", None)  # a sum that can be formed on the way
        if fused is not None and fused(ctx, h, rms[0], rms[1], weight, eps, rows, out):
            return True
        ops.add_normed_rmsnorm(h, self.tensor(ctx), rms[0], rms[1], weight, out, eps, rows)
        return True


register_part("norm", "rmsnorm", RMSNorm)
