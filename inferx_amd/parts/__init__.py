"""Parts a layer is put together from; importing this package registers the built-in ones."""
from .base import (Block, CacheNeed, FeedForward, LazyDelta, Mixer, Norm, ParamSpec, Part, PositionEncoding,
                   StateNeed, build_block, build_part, register_part, resolve_delta)
from . import norm, rope, dense_mlp, attention, moe, block  # noqa: F401  (registration)
from .model import DecoderModel, build_model

__all__ = ["Block", "CacheNeed", "FeedForward", "Mixer", "Norm", "ParamSpec", "Part", "PositionEncoding",
           "StateNeed", "LazyDelta", "resolve_delta", "build_block", "build_part", "register_part", "DecoderModel", "build_model"]
