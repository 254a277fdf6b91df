"""Random weights: a model folder (config.json + model.safetensors) from a
configuration and a seed, or tensors drawn directly on the device.

Every matrix and bias is normal with the configuration's standard deviation,
norm weights are one.  Each tensor has its own generator seeded from (seed,
tensor name), so a tensor's values do not depend on which other tensors exist.
Values are drawn in float32 and rounded to the storage type, so a bfloat16
folder and a float32 folder of one seed differ only by that rounding.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict

import torch

from .safetensors_io import write_safetensors


def _seed_for(seed: int, name: str) -> int:
    return (int(seed) * 0x9E3779B1 + zlib.crc32(name.encode("utf-8"))) % (2 ** 63 - 1)


def _storage_dtype(name: str) -> torch.dtype:
    try:
        return {"bfloat16": torch.bfloat16, "float32": torch.float32}[name]
    except KeyError:
        raise ValueError(f"storage dtype {name!r} is not bfloat16 or float32") from None


def random_tensors(model, seed: int, dtype: str = "bfloat16", device: str = "cpu") -> Dict[str, torch.Tensor]:
    store = _storage_dtype(dtype)
    out = {}
    for name, p in model.expected_tensors().items():
        if p.init == "ones":
            t = torch.ones(p.shape, dtype=torch.float32, device=device)
        elif p.init == "zeros":
            t = torch.zeros(p.shape, dtype=torch.float32, device=device)
        elif p.init == "normal":
            gen = torch.Generator(device=device)
            gen.manual_seed(_seed_for(seed, name))
            t = torch.randn(p.shape, dtype=torch.float32, device=device, generator=gen) * p.std
        else:
            raise ValueError(f"tensor {name!r}: unknown init {p.init!r}")
        out[name] = t.to(store)
    return out


def write_model_folder(config, seed: int, out_dir: str, dtype: str = "bfloat16") -> str:
    """config.json and model.safetensors for `config` with random weights."""
    from ..parts import build_model
    os.makedirs(out_dir, exist_ok=True)
    model = build_model(config.model_spec())
    raw = config.to_dict()
    raw["torch_dtype"] = dtype
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(raw, f, indent=2, sort_keys=True)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), random_tensors(model, seed, dtype))
    return out_dir
