"""A decoder model put together from a `ModelSpec`: embedding, layers in the
order of the schedule, final norm, head.  Nothing here names an architecture.

    logits = head( final_norm( run of blocks( embed(ids) ) )[wanted rows] )

Only the wanted rows go through the final norm and the head (the reference
computes all rows and picks afterwards, src/model/qwen2.cc:1059-1066).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .. import ops
from ..config.spec import ModelSpec, PartSpec
from .base import CacheNeed, ParamSpec, StateNeed, build_block, build_part


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.blocks = []
        self._part_specs: List[Tuple[PartSpec, object]] = []  # (spec, part) for every part that has tensors
        for layer in spec.layers:
            mixer = build_part("mixer", layer.mixer)
            ffn = build_part("feed_forward", layer.feed_forward)
            n1 = build_part("norm", layer.mixer_norm)
            n2 = build_part("norm", layer.feed_forward_norm)
            self.blocks.append(build_block(layer.block, mixer, ffn, n1, n2))
            self._part_specs += [(layer.mixer, mixer), (layer.feed_forward, ffn), (layer.mixer_norm, n1),
                                 (layer.feed_forward_norm, n2)]
        self.final_norm = build_part("norm", spec.final_norm)
        self._part_specs.append((spec.final_norm, self.final_norm))
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None

    # ---- tensors ---------------------------------------------------------
    def expected_tensors(self) -> Dict[str, ParamSpec]:
        """Checkpoint name -> what must be there (shape, and how to draw it at random)."""
        s = self.spec
        out: Dict[str, ParamSpec] = {
            s.embedding_name: ParamSpec(s.embedding_name, (s.vocab_size, s.hidden_size), std=s.init_std)}
        if s.head_name is not None:
            out[s.head_name] = ParamSpec(s.head_name, (s.vocab_size, s.hidden_size), std=s.init_std)
        for pspec, part in self._part_specs:
            for p in part.param_specs():
                name = pspec.tensor_name(p.name)
                if name in out and out[name].shape != tuple(p.shape):
                    raise ValueError(f"tensor {name!r} is claimed twice with different shapes")
                out[name] = p
        return out

    def bind(self, weights: Dict[str, torch.Tensor], rt) -> None:
        """Hand every part its tensors (already on the device).  `weights` is emptied."""
        s = self.spec
        self.embedding = weights[s.embedding_name].contiguous()
        self.head = weights[s.head_name].contiguous() if s.head_name is not None else self.embedding
        for pspec, part in self._part_specs:
            local = {p.name: weights[pspec.tensor_name(p.name)] for p in part.param_specs()}
            part.bind(local, rt)
        weights.clear()

    def graph_safe(self) -> bool:
        """True if every part may run inside a captured HIP graph."""
        parts = [self.final_norm]
        for b in self.blocks:
            parts += [b, b.mixer, b.feed_forward, b.mixer_norm, b.feed_forward_norm]
            parts.append(getattr(b.mixer, "position", None))
        return all(getattr(p, "graph_safe", False) for p in parts if p is not None)

    # ---- what the cache manager must provide -------------------------------
    def cache_plan(self):
        """Per schedule entry: (CacheNeed or None, StateNeed or None, cache_from)."""
        plan = []
        for entry in self.spec.schedule:
            mixer = self.blocks[entry.layer].mixer
            plan.append((mixer.cache_need(), mixer.state_need(), entry.cache_from))
        return plan

    # ---- one step ----------------------------------------------------------
    def forward(self, ctx, caches) -> torch.Tensor:
        """caches: one CacheBinding per schedule entry.  Returns float32 [R, vocab]."""
        s = self.spec
        h = ctx.rt.empty((ctx.num_tokens, s.hidden_size), torch.float32)
        ops.embed(h, self.embedding, ctx.token_ids)
        pending = None
        for i, entry in enumerate(s.schedule):
            pending = self.blocks[entry.layer].forward(ctx, h, pending, caches[i])
        rows = ctx.logits_rows
        if rows.numel() == 0:
            return ctx.rt.empty((0, s.vocab_size), torch.float32)
        x = self.final_norm.forward(ctx, h, pending, rows=rows)
        return ctx.rt.linear_f32(x, self.head)


def build_model(spec: ModelSpec) -> DecoderModel:
    return DecoderModel(spec)
