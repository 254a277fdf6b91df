"""Typed configurations and the architecture registry."""
from .registry import (ConfigError, config_class_for, config_from_dict, config_from_directory,
                       config_from_json, known_architectures, register_architecture)
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding
from . import qwen2_moe  # registers Qwen2MoeForCausalLM
from .qwen2_moe import Qwen2MoeConfig

__all__ = [
    "ConfigError", "config_class_for", "config_from_dict", "config_from_directory", "config_from_json",
    "known_architectures", "register_architecture", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry", "linear_head", "token_embedding",
    "Qwen2MoeConfig",
]
