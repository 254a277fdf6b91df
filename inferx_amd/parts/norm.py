"""RMSNorm, fused with the residual add that precedes it.

y = v * rsqrt(mean(v^2) + eps) * weight with v = h + delta, everything in
float32, rounded once (reference: RmsNormKernel, src/backends/cuda/ops/layers.cu:50-76).
"""
from __future__ import annotations

from typing import List

from .. import ops
from .base import LazyDelta, Norm, ParamSpec, register_part


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, width: int, eps: float):
        self.width, self.eps = int(width), float(eps)
        self.weight = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.width,), init="ones")]

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].contiguous()

    def rms_operands(self):
        return self.weight, self.eps

    def forward(self, ctx, h, delta=None, rows=None):
        """h [T, width] float32 is updated in place with `delta` (unless `rows`
        picks rows out); returns the normalised rows in the run's type."""
        n = h.shape[0] if rows is None else rows.numel()
        out = ctx.rt.empty((n, self.width))
        if isinstance(delta, LazyDelta):
            if delta.add_rmsnorm(ctx, h, self.weight, self.eps, rows, out):
                return out
            delta = delta.materialize(ctx)
        ops.add_rmsnorm(h, delta, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
