"""Binding a checkpoint's tensors to a model by name.

The model says what it needs (`DecoderModel.expected_tensors`); the loader
compares that with what the folder holds and raises ONE error that lists every
missing tensor, every unexpected one and every wrong shape (the reference
reports them one at a time: NotFound `src/model/safetensors.cc:389-392`, shape
mismatch `:417-421`).  Tensors keep their stored floating type in a bfloat16
run (bfloat16 stays, 32-bit stays 32-bit) and all become float32 in a float32
run; integer tables become int32.
"""
from __future__ import annotations

from typing import Dict, List, Sequence

import torch

from .safetensors_io import Checkpoint, CheckpointError


def check_names_and_shapes(expected: Dict[str, tuple], ckpt: Checkpoint, ignored_suffixes: Sequence[str] = ()) -> None:
    """`ignored_suffixes`: endings of tensor names that a checkpoint of this architecture may hold although no part
    asks for them (the model's spec lists them)."""
    missing: List[str] = sorted(n for n in expected if n not in ckpt)
    ignored = tuple(ignored_suffixes)
    unexpected = sorted(n for n in ckpt.names() if n not in expected and not (ignored and n.endswith(ignored)))
    wrong = sorted(
        f"{n}: expected {list(expected[n])}, file has {list(ckpt.shape(n))}"
        for n in expected if n in ckpt and tuple(ckpt.shape(n)) != tuple(expected[n]))
    bad_type = sorted(f"{n}: {ckpt.dtype(n)}" for n in expected
                      if n in ckpt and not ckpt.dtype(n).is_floating_point)
    if not (missing or unexpected or wrong or bad_type):
        return

    def block(title, items):
        if not items:
            return ""
        shown = items[:40]
        more = f"\n    ... and {len(items) - 40} more" if len(items) > 40 else ""
        return f"\n  {title} ({len(items)}):\n    " + "\n    ".join(shown) + more

    raise CheckpointError(
        "the checkpoint does not fit the model:"
        + block("missing tensors", missing) + block("unexpected tensors", unexpected)
        + block("wrong shapes", wrong) + block("not floating point", bad_type))


def load_weights(model, model_dir: str, rt) -> Dict[str, torch.Tensor]:
    """All tensors the model needs, on the device, keyed by checkpoint name."""
    ckpt = Checkpoint.open(model_dir)
    expected = {name: tuple(p.shape) for name, p in model.expected_tensors().items()}
    check_names_and_shapes(expected, ckpt, model.spec.ignored_tensor_suffixes)
    return {name: rt.place(ckpt.get(name)) for name in expected}
