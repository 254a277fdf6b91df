"""Rotary position encoding, half-split pairing (j, j + d/2).

f_j = theta^(-2j/d), angle = position * f_j; the rotation itself is fused into
the kernel that follows the q/k/v product (reference: RopeKernel,
src/backends/cuda/ops/layers.cu:80-115; ops/layers.h:35-58).  The frequencies
are computed once in float64 and rounded to float32; the angle and its cosine
and sine are float32, once per step for all layers.

Interface of a position encoding: `prepare(ctx)` returns a float32 table
[T, rotary_dim/2, 2] of (cos, sin) for this step's tokens, or None for no
rotation.  An encoding that rotates only a part of each head says so with its
attributes `rotary_dim` (how many elements) and `begin` (the first of them;
0 if absent): the elements outside pass through (the reference's own partial
rotation takes the trailing part of a head, src/backends/cuda/ops/mla.cu:24-46).
"""
from __future__ import annotations

import torch

from .. import ops
from .base import PositionEncoding, register_part


class Rotary(PositionEncoding):
    graph_safe = True

    def __init__(self, theta: float, rotary_dim: int, begin: int = 0):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary_dim {rotary_dim} must be positive and even")
        if theta <= 0:
            raise ValueError("theta must be positive")
        if begin < 0:
            raise ValueError("the rotated part cannot begin before the head")
        self.theta, self.rotary_dim, self.begin = float(theta), int(rotary_dim), int(begin)
        self.inv_freq = None

    def frequencies(self) -> torch.Tensor:
        j = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        return torch.pow(torch.tensor(self.theta, dtype=torch.float64), -2.0 * j / self.rotary_dim).to(torch.float32)

    def bind(self, tensors, rt) -> None:
        self.inv_freq = self.frequencies().to(rt.device)

    def prepare(self, ctx):
        key = ("rope", self.theta, self.rotary_dim)
        table = ctx.memo.get(key)
        if table is None:
            table = ctx.rt.empty((ctx.num_tokens, self.rotary_dim // 2, 2), torch.float32)
            ops.rope_table(table, ctx.positions, self.inv_freq)
            ctx.memo[key] = table
        return table


register_part("position", "rope", Rotary)
