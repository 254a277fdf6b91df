"""A decoder model put together from a `ModelSpec`: embedding, layers in the
order of the schedule, final norm, head.  Nothing here names an architecture.

    logits = head( final_norm( run of blocks( embedding(ids) ) )[wanted rows] )

Only the wanted rows go through the final norm and the head (the reference
computes all rows and picks afterwards, src/model/qwen2.cc:1059-1066).  Both
ends are parts like the others: an architecture that scales its embeddings,
adds learned positions or caps its logits registers an embedding or a head of
its own.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from .base import CacheNeed, ParamSpec, Part, StateNeed, build_block, build_part


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.blocks = []
        self._part_specs: List[Tuple[PartSpec, Part]] = []  # (spec, part) for every part built from a spec
        self.embedding = build_part("embedding", spec.embedding)
        self._part_specs.append((spec.embedding, self.embedding))
        for layer in spec.layers:
            block = build_block(layer.block, layer.parts)
            self.blocks.append(block)
            self._part_specs += [(layer.parts[name], block.parts[name]) for name in layer.parts]
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self._part_specs += [(spec.final_norm, self.final_norm), (spec.head, self.head)]

    # ---- tensors ---------------------------------------------------------
    def expected_tensors(self) -> Dict[str, ParamSpec]:
        """Checkpoint name -> what must be there (shape, and how to draw it at random).  Two parts may name the
        same tensor (a head tied to the embedding) if they agree on its shape."""
        out: Dict[str, ParamSpec] = {}
        for pspec, part in self._part_specs:
            for p in part.param_specs():
                name = pspec.tensor_name(p.name)
                if name in out and tuple(out[name].shape) != tuple(p.shape):
                    raise ValueError(f"tensor {name!r} is claimed twice with different shapes")
                out.setdefault(name, p)
        return out

    def shared_tensor_names(self) -> List[str]:
        """Checkpoint names that more than one part claims (a head tied to the embedding)."""
        seen: Dict[str, int] = {}
        for pspec, part in self._part_specs:
            for p in part.param_specs():
                name = pspec.tensor_name(p.name)
                seen[name] = seen.get(name, 0) + 1
        return [n for n, c in seen.items() if c > 1]

    def bind(self, weights, rt) -> None:
        """Hand every part its tensors: `weights` maps checkpoint names to tensors on the device (a dict, or a
        mapping that fetches each when it is asked for) and is emptied."""
        for pspec, part in self._part_specs:
            local = {p.name: weights[pspec.tensor_name(p.name)] for p in part.param_specs()}
            part.bind(local, rt)
        weights.clear()

    def all_parts(self) -> List[Part]:
        """Every part of the model, the blocks and the parts' own sub-parts included."""
        out: List = [self.embedding, self.final_norm, self.head]
        for b in self.blocks:
            out.append(b)
            out += list(b.parts.values())
        for p in list(out):
            out += [s for s in getattr(p, "subparts", lambda: [])() if s is not None]
        return out

    def graph_safe(self) -> bool:
        """True if every part may run inside a captured HIP graph."""
        return all(getattr(p, "graph_safe", False) for p in self.all_parts())

    # ---- what the cache manager must provide -------------------------------
    def cache_plan(self):
        """Per schedule entry: ({part name: (CacheNeed or None, StateNeed or None)} for the parts of the layer that
        keep something between steps, cache_from)."""
        plan = []
        for entry in self.spec.schedule:
            keeps: Dict[str, Tuple[Optional[CacheNeed], Optional[StateNeed]]] = {}
            for name, part in self.blocks[entry.layer].parts.items():
                need, state = part.cache_need(), part.state_need()
                if need is not None or state is not None:
                    keeps[name] = (need, state)
            plan.append((keeps, entry.cache_from))
        return plan

    # ---- one step ----------------------------------------------------------
    def forward(self, ctx, caches) -> torch.Tensor:
        """caches: per schedule entry, the `CacheBinding`s of its parts by name.  Returns float32 [R, vocab]."""
        s = self.spec
        h = self.embedding.forward(ctx)
        pending = None
        for i, entry in enumerate(s.schedule):
            pending = self.blocks[entry.layer].forward(ctx, h, pending, caches[i])
        rows = ctx.logits_rows
        if rows.numel() == 0:
            return ctx.rt.empty((0, s.vocab_size), torch.float32)
        x = self.final_norm.forward(ctx, h, pending, rows=rows)
        return self.head.forward(ctx, x)


def build_model(spec: ModelSpec) -> DecoderModel:
    return DecoderModel(spec)
