"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from the parameters in its `PartSpec`, never from a config
object, and does not know which model it is in.  Five kinds:

  Norm              forward(ctx, h, delta=None, rows=None) -> normed activations
  PositionEncoding  prepare(ctx) -> whatever its mixer's kernels need this step
  Mixer             forward(ctx, x, cache) -> delta   (attention here)
  FeedForward       forward(ctx, x) -> delta          (dense or experts)
  Block             forward(ctx, h, pending, layer, cache) -> pending delta

Every part lists the tensors it needs (`param_specs`) under local names; the
`PartSpec` maps those to checkpoint names.  `bind` receives the loaded tensors
(on the device, in their stored floating type or the run's type) and may fuse
them (q/k/v rows stacked, experts stacked).

A mixer also says what it keeps between steps: `cache_need()` (pages of keys
and values, all of them or a window) and `state_need()` (a block of fixed size
per request).
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
class CacheNeed:
    """Keys and values in pages.  `window` 0: all earlier tokens are read; W > 0:
    only the last W (the query's own included), so older pages may be given back.
    Entries with equal needs share a group of pages."""

    kv_heads: int
    head_dim: int
    window: int = 0


@dataclass(frozen=True)
class StateNeed:
    """A block of `shape` float32 numbers per request, zero when a request starts."""

    shape: Tuple[int, ...]


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
    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, ctx, x, cache):
        raise NotImplementedError


class FeedForward(Part):
    takes_lazy_norm = False  # True: `x` may be a LazyNorm (see there)

    def forward(self, ctx, x):
        raise NotImplementedError


class Block:
    graph_safe = False

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def forward(self, ctx, h, pending, cache):
        raise NotImplementedError


_REGISTRIES: Dict[str, Dict[str, Callable[..., Any]]] = {
    "norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "block": {},
}


def register_part(kind: str, name: str, factory: Callable[..., Any]) -> None:
    """kind: 'norm' | 'position' | 'mixer' | 'feed_forward' | 'block'."""
    if kind not in _REGISTRIES:
        raise KeyError(f"no such kind of part: {kind!r} (known: {', '.join(_REGISTRIES)})")
    _REGISTRIES[kind][name] = factory


def build_part(kind: str, spec: PartSpec):
    reg = _REGISTRIES[kind]
    if spec.kind not in reg:
        raise KeyError(f"no {kind} registered as {spec.kind!r} (known: {', '.join(sorted(reg)) or '(none)'})")
    return reg[spec.kind](**spec.params)


def build_block(name: str, mixer, feed_forward, mixer_norm, feed_forward_norm) -> Block:
    reg = _REGISTRIES["block"]
    if name not in reg:
        raise KeyError(f"no block registered as {name!r} (known: {', '.join(sorted(reg)) or '(none)'})")
    return reg[name](mixer, feed_forward, mixer_norm, feed_forward_norm)
