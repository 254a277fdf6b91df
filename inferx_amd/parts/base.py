"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from the parameters in its `PartSpec`, never from a config
object, and does not know which model it is in.  Seven kinds:

  Embedding         forward(ctx) -> the residual stream h, float32 [T, hidden]
  Norm              forward(ctx, h, delta=None, rows=None) -> normed activations
  PositionEncoding  prepare(ctx) -> whatever its mixer's kernels need this step
  Mixer             forward(ctx, x, cache) -> delta   (attention here)
  FeedForward       forward(ctx, x) -> delta          (dense or experts)
  Block             forward(ctx, h, pending, caches) -> pending delta; names the parts it arranges
  Head              forward(ctx, x) -> float32 logits [rows, vocab]

Every part lists the tensors it needs (`param_specs`) under local names; the
`PartSpec` maps those to checkpoint names.  `bind` receives the loaded tensors
(on the device, in their stored floating type or the run's type) and may fuse
them (q/k/v rows stacked, experts stacked).

Any part may keep something between steps and says so: `cache_need()` (arrays
in pages, one entry per token: all tokens or a window of them) and
`state_need()` (a block of fixed size per request).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Tuple

from ..config.spec import PartSpec


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part needs.  `init`: 'normal' (std = `std`), 'ones' or 'zeros'."""

    name: str
    shape: Tuple[int, ...]
    init: str = "normal"
    std: float = 0.02


@dataclass(frozen=True)
class CacheArray:
    """One array that a part keeps per token, in pages: `heads` x `width` numbers per token.  Laid out
    [pages, heads, page_size, width], or with `transposed` [pages, heads, width, page_size] (a page's tokens
    contiguous per column).  `dtype` None: the run's type; else "float32" or "bfloat16".
    (The reference's `KvLayout{entries_per_token, kv_heads, head_dim, dtype}`, include/inferx/core/kv_cache.h:14-38.)"""

    name: str
    heads: int
    width: int
    transposed: bool = False
    dtype: Optional[str] = None


@dataclass(frozen=True)
class CacheNeed:
    """What a part keeps per token, in pages: the arrays it names, for all earlier tokens (`window` 0) or only
    the last W (the query's own included), so that older pages may be given back.  Parts with equal needs share a
    group of pages (one pool, one block table per request); the runner allocates each array from this description
    and knows nothing else about it."""

    arrays: Tuple[CacheArray, ...]
    window: int = 0

    @staticmethod
    def keys_and_values(kv_heads: int, head_dim: int, window: int = 0) -> "CacheNeed":
        """Attention's cache: keys [pages, kv_heads, page_size, head_dim] and values transposed within a page."""
        return CacheNeed((CacheArray("k", kv_heads, head_dim), CacheArray("v", kv_heads, head_dim, transposed=True)),
                         window)


@dataclass(frozen=True)
class StateNeed:
    """A block of `shape` numbers per request ("float32", "bfloat16", "int32" or "int64"), zero when a request
    starts."""

    shape: Tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self):
        if self.dtype not in ("float32", "bfloat16", "int32", "int64"):
            raise ValueError(f"per-request state of type {self.dtype!r}: float32, bfloat16, int32 or int64")


class LazyDelta:
    """What a mixer or feed-forward may return instead of a tensor: a delta that is not formed yet, so that the
    norm that consumes it can form it, add it to the residual stream and normalise in one kernel.
    A norm that cannot do that calls `materialize` and goes on with the tensor."""

    def materialize(self, ctx):
        raise NotImplementedError

    def add_rmsnorm(self, ctx, h, weight, eps, rows, out) -> bool:
        """h += delta; out = rmsnorm(h) * weight.  Returns False if this case is not fused (then nothing was done)."""
        return False


def resolve_delta(ctx, delta):
    """A tensor (or None) whatever `delta` is."""
    return delta.materialize(ctx) if isinstance(delta, LazyDelta) else delta


class LazyNorm:
    """What a block may hand to a feed-forward that says `takes_lazy_norm`, instead of the normalised tensor: the
    norm and its operands, not applied yet, so that the feed-forward's first kernel can apply it (and update the
    residual stream) on its way.  A feed-forward that does not fuse this case calls `materialize` and goes on
    with the tensor; either way h has had `delta` added when the feed-forward returns."""

    def __init__(self, norm, h, delta):
        self.norm, self.h, self.delta = norm, h, delta

    def materialize(self, ctx):
        return self.norm.forward(ctx, self.h, self.delta)

    def rms_operands(self):
        """(weight, eps) if the norm is y = v * rsqrt(mean(v^2) + eps) * weight and `delta` is a tensor, else None."""
        if isinstance(self.delta, LazyDelta) or self.delta is None:
            return None
        return self.norm.rms_operands()


def resolve_input(ctx, x):
    """A tensor whatever `x` is."""
    return x.materialize(ctx) if isinstance(x, LazyNorm) else x


class Part:
    # True if `forward` only launches work on the current stream (no host reads of device data, no host-side
    # planning from the batch), so that a step can be captured into a HIP graph
    graph_safe = False

    def param_specs(self) -> List[ParamSpec]:
        return []

    def bind(self, tensors: Dict[str, Any], rt) -> None:
        """Take ownership of the loaded tensors (keys: local names)."""

    def subparts(self) -> List["Part"]:
        """Parts this part built for itself (a mixer's position encoding)."""
        return []

    # ---- what the part keeps between steps (nothing unless it says so) ----
    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    # ---- steps of one token per request that are replayed from a graph ----
    def capture_plan(self, ctx, requests: int, longest: int) -> None:
        """A part that plans on the host (`ctx.host`) leaves here, in `ctx.memo`, whatever its `forward` looks up
        when `ctx.host` is None: the plan of a step in which each of `requests` requests brings one token and no
        context is longer than `longest`.  The plan must not depend on anything else, because the recorded step is
        replayed for every such batch.  The runner calls this for every part before it records such a step, and
        before it runs one kernel by kernel too, so that both ways make the same choices."""


class Norm(Part):
    def rms_operands(self):
        """(weight, eps) if this is a plain RMS norm that another kernel may apply, else None."""
        return None

    def forward(self, ctx, h, delta=None, rows=None):
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, ctx):
        raise NotImplementedError


class Mixer(Part):
    def forward(self, ctx, x, cache):
        """`cache`: the `CacheBinding` of this execution (its arrays of pages, its state), or None if the mixer
        keeps nothing."""
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ctx):
        """The residual stream for this step's tokens: float32 [T, hidden]."""
        raise NotImplementedError


class Head(Part):
    def forward(self, ctx, x):
        """x: the normalised wanted rows in the run's type; returns float32 logits [rows, vocab]."""
        raise NotImplementedError


class FeedForward(Part):
    takes_lazy_norm = False  # True: `x` may be a LazyNorm (see there)

    def forward(self, ctx, x):
        raise NotImplementedError


class Block:
    """An arrangement of parts around the residual stream.  `part_kinds` names the parts the arrangement needs
    and the kind of each (a key of the registries); names in `optional_parts` may be left out of a `LayerSpec`.
    The parts arrive built, by name, and are also set as attributes.  `caches` in `forward` holds, by part name,
    the `CacheBinding` of every part of this execution that keeps pages or state."""

    graph_safe = False
    part_kinds: Dict[str, str] = {}
    optional_parts: Tuple[str, ...] = ()

    def __init__(self, parts: Dict[str, Part]):
        self.parts = dict(parts)
        for name in self.part_kinds:
            setattr(self, name, self.parts.get(name))

    def forward(self, ctx, h, pending, caches):
        raise NotImplementedError


_REGISTRIES: Dict[str, Dict[str, Callable[..., Any]]] = {
    "norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(kind: str, name: str, factory: Callable[..., Any]) -> None:
    """kind: 'norm' | 'position' | 'mixer' | 'feed_forward' | 'block' | 'embedding' | 'head'.  A block is
    registered by its class (see `Block`), every other kind by a callable that takes the `PartSpec`'s parameters."""
    if kind not in _REGISTRIES:
        raise KeyError(f"no such kind of part: {kind!r} (known: {', '.join(_REGISTRIES)})")
    _REGISTRIES[kind][name] = factory


def build_part(kind: str, spec: PartSpec):
    reg = _REGISTRIES[kind]
    if spec.kind not in reg:
        raise KeyError(f"no {kind} registered as {spec.kind!r} (known: {', '.join(sorted(reg)) or '(none)'})")
    return reg[spec.kind](**spec.params)


def build_block(name: str, part_specs: Dict[str, PartSpec]) -> Block:
    """The arrangement `name` with its parts built from their specs; a part the arrangement does not know, or one
    it needs and does not get, is an error that names it."""
    reg = _REGISTRIES["block"]
    if name not in reg:
        raise KeyError(f"no block registered as {name!r} (known: {', '.join(sorted(reg)) or '(none)'})")
    cls = reg[name]
    kinds = cls.part_kinds
    unknown = sorted(set(part_specs) - set(kinds))
    missing = sorted(set(kinds) - set(part_specs) - set(cls.optional_parts))
    if unknown or missing:
        raise KeyError(f"block {name!r} arranges the parts {sorted(kinds)}: " +
                       "; ".join(([f"not known to it: {unknown}"] if unknown else []) +
                                 ([f"missing: {missing}"] if missing else [])))
    return cls({n: build_part(kinds[n], spec) for n, spec in part_specs.items()})
