"""The two ends of a model: token ids -> residual stream, and wanted rows -> logits.

h[t] = table[id_t] * scale (reference: EmbeddingKernel, src/backends/cuda/ops/layers.cu:465-481, no scale there);
logits = x . W^T in float32 for the wanted rows only (reference: src/model/qwen2.cc:1059-1066 computes all rows
and picks afterwards; a tied head aliases the table, :1335-1336: here the head's tensor simply carries the
embedding's checkpoint name, so both parts are handed the same tensor).
"""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from .base import Embedding, Head, ParamSpec, register_part


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, init_std: float = 0.02):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.scale, self.init_std = float(scale), float(init_std)
        self.weight = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.vocab_size, self.hidden_size), std=self.init_std)]

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, ctx):
        h = ctx.rt.empty((ctx.num_tokens, self.hidden_size), torch.float32)
        ops.embed(h, self.weight, ctx.token_ids, self.scale)
        return h


class LinearHead(Head):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, init_std: float = 0.02):
        self.vocab_size, self.hidden_size, self.init_std = int(vocab_size), int(hidden_size), float(init_std)
        self.weight = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec("weight", (self.vocab_size, self.hidden_size), std=self.init_std)]

    def bind(self, tensors, rt) -> None:
        self.weight = tensors["weight"].contiguous()

    def forward(self, ctx, x):
        return ctx.rt.linear_f32(x, self.weight)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "linear_head", LinearHead)
