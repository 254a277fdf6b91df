"""Weights: safetensors by tensor name, and the random-weights mode."""
from .safetensors_io import Checkpoint, CheckpointError, write_safetensors
from .loader import check_names_and_shapes, load_weights
from .random_init import random_tensors, write_model_folder

__all__ = ["Checkpoint", "CheckpointError", "write_safetensors", "check_names_and_shapes", "load_weights",
           "random_tensors", "write_model_folder"]
