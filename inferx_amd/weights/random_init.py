"""Random weights: a model folder (config.json + model.safetensors) from a
configuration and a seed, or tensors drawn directly on the device.

Every matrix and bias is normal with the configuration's standard deviation,
norm weights are one.  A value is a pure function of (seed, tensor name, element
index): a counter-based generator in integer arithmetic that gives the same bits
on the host and on the device, so a tensor's values do not depend on which
other tensors exist or where they are drawn, and the weights that a benchmark
draws on the device can be drawn again on the host.  Values are formed in
float32 and rounded to the storage type, so a bfloat16 folder and a float32
folder of one seed differ only by that rounding.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict

import torch

from .safetensors_io import write_safetensors


_MASK64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_CHUNK = 1 << 24  # elements formed at a time (a few hundred megabytes of 64-bit intermediates)


def _signed(v: int) -> int:
    """A 64-bit pattern as the int64 that holds it."""
    v &= _MASK64
    return v - (1 << 64) if v >> 63 else v


def _mix_int(z: int) -> int:
    """splitmix64's finaliser on a Python integer."""
    z &= _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)


def _mix(z: torch.Tensor) -> torch.Tensor:
    """The same on int64 tensors: products wrap round as 64-bit products do, and the right shifts are made logical
    by masking the sign bits that an arithmetic shift brings in.  Integer operations only, so host and device agree."""
    z = (z ^ ((z >> 30) & ((1 << 34) - 1))) * _signed(0xBF58476D1CE4E5B9)
    z = (z ^ ((z >> 27) & ((1 << 37) - 1))) * _signed(0x94D049BB133111EB)
    return z ^ ((z >> 31) & ((1 << 33) - 1))


def _key_for(seed: int, name: str) -> int:
    return _mix_int(_mix_int(int(seed)) ^ (zlib.crc32(name.encode("utf-8")) * _GOLDEN))


def counter_normal(seed: int, name: str, shape, std: float, device="cpu") -> torch.Tensor:
    """float32 values of standard deviation `std`: element i is a function of (seed, name, i) alone.  Three 64-bit
    hashes of the element's counter give twelve 16-bit numbers; their sum, centred and scaled, is (to a good
    approximation, within six standard deviations) normal.  The sum is an integer below 2^20, the centring and the
    division by 2^16 are exact in float32, and the one rounding is that of the product with `std`."""
    n = 1
    for d in shape:
        n *= int(d)
    out = torch.empty(n, dtype=torch.float32, device=device)
    key = _key_for(seed, name)
    for start in range(0, n, _CHUNK):
        stop = min(n, start + _CHUNK)
        counter = torch.arange(start, stop, dtype=torch.int64, device=device) * 3
        total = torch.zeros(stop - start, dtype=torch.int64, device=device)
        for j in range(3):
            h = _mix((counter + j) * _signed(_GOLDEN) + _signed(key))
            for shift in (0, 16, 32, 48):
                total += (h >> shift) & 0xFFFF
        out[start:stop] = (total - 393210).to(torch.float32) * (1.0 / 65536.0) * float(std)
    return out.view(tuple(int(d) for d in shape))


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
            t = counter_normal(seed, name, p.shape, p.std, device)
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
