"""Parts a layer is put together from; importing this package registers the built-in ones."""
from .base import (Block, CacheArray, CacheNeed, Embedding, FeedForward, Head, LazyDelta, LazyNorm, Mixer, Norm, ParamSpec, Part,
                   PositionEncoding, StateNeed, build_block, build_part, register_part, resolve_delta, resolve_input)
from . import norm, rope, dense_mlp, attention, moe, block, embedding  # noqa: F401  (registration)
from .model import DecoderModel, build_model

__all__ = ["Block", "CacheArray", "CacheNeed", "Embedding", "Head", "FeedForward", "Mixer", "Norm", "ParamSpec", "Part", "PositionEncoding",
           "StateNeed", "LazyDelta", "LazyNorm", "resolve_delta", "resolve_input", "build_block", "build_part",
           "register_part", "DecoderModel", "build_model"]
