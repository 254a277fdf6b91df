"""Architecture-neutral description of a model: what an architecture's config
turns into, and what the builder, the loader, the random-weights writer and the
cache manager read.

A `ModelSpec` is plain data.  It names parts by the key under which they are
registered (`inferx_amd.parts.registry`) and carries their sizes and constants
as parameters; nothing below this file looks at an architecture's config keys.

The reference keeps one flat `ModelConfig` with per-layer predicates
(`include/inferx/model/config.h:48-252`, `IsMoeLayer` `:121-126`,
`IsSlidingLayer` `:196-203`); here the predicates are evaluated once, when the
config is turned into a list of `LayerSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: registry key, constructor parameters and where its
    tensors live in the checkpoint.

    `prefix` is put before each of the part's local tensor names; `rename`
    replaces a local name first (for an architecture that spells it
    differently)."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    prefix: str = ""
    rename: Dict[str, str] = field(default_factory=dict)

    def tensor_name(self, local: str) -> str:
        return self.prefix + self.rename.get(local, local)


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: how its parts are arranged (`block`) and the parts."""

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec


@dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer.  `layer` indexes `ModelSpec.layers` (a layer
    may be named by several entries: shared weights, separate caches).
    `cache_from` names an EARLIER entry whose cache this execution reads
    instead of owning one (it then writes nothing)."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    embedding_name: str
    final_norm: PartSpec
    head_name: Optional[str]  # None: the head is the embedding table (tied)
    init_std: float = 0.02

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ValueError("hidden_size and vocab_size must be positive")
        if not self.layers or not self.schedule:
            raise ValueError("a model needs at least one layer and one schedule entry")
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"schedule[{i}] names layer {e.layer}, model has {len(self.layers)}")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ValueError(f"schedule[{i}].cache_from={e.cache_from} must name an earlier entry")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ValueError(f"schedule[{i}].cache_from names an entry that owns no cache")
