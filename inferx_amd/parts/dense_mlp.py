"""Dense gated feed-forward: down( silu(gate(x)) * up(x) ).

gate and up are stacked into one [2I, H] matrix, gate rows first (reference:
src/model/qwen2.cc:1413-1434 load, :1042-1048 forward; SiluMulFusedKernel
layers.cu:512-529).
"""
from __future__ import annotations

from typing import List

import torch

from .base import FeedForward, ParamSpec, register_part


def stack_rows(tensors):
    """Concatenate along dim 0; mixed storage types widen to float32."""
    if len({t.dtype for t in tensors}) > 1:
        tensors = [t.to(torch.float32) for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


class DenseMlp(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, init_std: float = 0.02):
        self.hidden_size, self.width, self.init_std = int(hidden_size), int(width), float(init_std)
        self.w_gate_up = self.w_down = None

    def param_specs(self) -> List[ParamSpec]:
        H, I, s = self.hidden_size, self.width, self.init_std
        return [ParamSpec("gate_proj.weight", (I, H), std=s), ParamSpec("up_proj.weight", (I, H), std=s),
                ParamSpec("down_proj.weight", (H, I), std=s)]

    def bind(self, tensors, rt) -> None:
        self.w_gate_up = stack_rows([tensors["gate_proj.weight"], tensors["up_proj.weight"]])
        self.w_down = tensors["down_proj.weight"].contiguous()

    def forward(self, ctx, x):
        rt = ctx.rt
        return rt.linear(rt.gated_linear(x, self.w_gate_up), self.w_down)


register_part("feed_forward", "dense_mlp", DenseMlp)
