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

from collections.abc import Mapping
from typing import Callable, Dict, Iterable, Iterator, List, Sequence

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


class LazyWeights(Mapping):
    """The tensors a model needs, by checkpoint name, each brought to the device when it is asked for and not kept
    here: a part that restacks what it is given (the experts of a mixture, gate|up of a dense feed-forward) then
    holds its own layout only, and loading peaks at the size of the model plus one layer's tensors instead of
    twice the model.  A tensor that more than one part claims (a head tied to the embedding) is kept after its
    first use, so that all of them get the same one."""

    def __init__(self, names: Iterable[str], fetch: Callable[[str], torch.Tensor], shared: Iterable[str] = ()):
        self._names = list(names)
        self._known = set(self._names)
        self._fetch = fetch
        self._shared = set(shared)
        self._kept: Dict[str, torch.Tensor] = {}

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self._known:
            raise KeyError(name)
        if name in self._kept:
            return self._kept[name]
        t = self._fetch(name)
        if name in self._shared:
            self._kept[name] = t
        return t

    def __contains__(self, name) -> bool:  # (the inherited one would fetch the tensor to find out)
        return name in self._known

    def __iter__(self) -> Iterator[str]:
        return iter(self._names)

    def __len__(self) -> int:
        return len(self._names)

    def clear(self) -> None:
        self._names, self._known, self._kept = [], set(), {}


def load_weights(model, model_dir: str, rt) -> Mapping:
    """All tensors the model needs, keyed by checkpoint name; each is read and put on the device when the model's
    `bind` asks for it (`LazyWeights`).  Names, shapes and types are checked here, before anything is read."""
    ckpt = Checkpoint.open(model_dir)
    expected = {name: tuple(p.shape) for name, p in model.expected_tensors().items()}
    check_names_and_shapes(expected, ckpt, model.spec.ignored_tensor_suffixes)
    return LazyWeights(expected, lambda name: rt.place(ckpt.get(name)), model.shared_tensor_names())
