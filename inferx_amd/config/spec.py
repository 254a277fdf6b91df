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
from typing import Any, Dict, List, Optional, Tuple


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
    """One decoder layer: how its parts are arranged (`block`, a registered arrangement) and the parts themselves
    under the names that arrangement gives them.  The arrangement says which names it needs and of which kind
    each is ("prenorm": mixer, feed_forward, mixer_norm, feed_forward_norm); another arrangement may want more
    norms, fewer, or two mixers, without a change here."""

    block: str
    parts: Dict[str, PartSpec]


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
    """`embedding` (kind "embedding") turns the step's token ids into the residual stream, `final_norm` (kind
    "norm") and `head` (kind "head") turn the wanted rows of the stream into logits.  A head that shares the
    embedding's table names the same checkpoint tensor through its `rename`."""

    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    embedding: PartSpec
    final_norm: PartSpec
    head: PartSpec
    init_std: float = 0.02
    # endings of tensor names that a checkpoint may hold although no part reads them (tables some writers add, the
    # head's copy of a tied embedding)
    ignored_tensor_suffixes: Tuple[str, ...] = ()

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


def token_embedding(name: str, vocab_size: int, hidden_size: int, init_std: float = 0.02,
                    scale: float = 1.0) -> PartSpec:
    """The usual embedding: one table `name` of [vocab, hidden]."""
    return PartSpec("token_embedding", {"vocab_size": vocab_size, "hidden_size": hidden_size, "scale": scale,
                                        "init_std": init_std}, rename={"weight": name})


def linear_head(name: str, vocab_size: int, hidden_size: int, init_std: float = 0.02) -> PartSpec:
    """The usual head: logits = x . W^T with W = `name` of [vocab, hidden]; a tied head names the embedding's table."""
    return PartSpec("linear_head", {"vocab_size": vocab_size, "hidden_size": hidden_size, "init_std": init_std},
                    rename={"weight": name})
