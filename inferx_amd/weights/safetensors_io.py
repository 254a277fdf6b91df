"""Reading and writing the safetensors container, by tensor name.

Format (reference: `src/model/safetensors.cc:20-23, 157-277`): an unsigned 64-bit
little-endian header length, a JSON object `{name: {dtype, shape, data_offsets:
[begin, end]}}` (the key `__metadata__` is skipped), then the data; offsets count
from the end of the header.  Sharded checkpoints are found through
`model.safetensors.index.json` (`weight_map`, `safetensors.cc:286-331`).

The file is memory-mapped; a tensor is handed out as a torch tensor that views
the map (bfloat16 through a 16-bit integer view), so nothing is copied until
the caller moves it to the device.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch

MAX_HEADER_BYTES = 256 << 20

_DTYPES = {
    "F64": (torch.float64, np.float64, 8),
    "F32": (torch.float32, np.float32, 4),
    "F16": (torch.float16, np.float16, 2),
    "BF16": (torch.bfloat16, np.uint16, 2),
    "I64": (torch.int64, np.int64, 8),
    "I32": (torch.int32, np.int32, 4),
    "I16": (torch.int16, np.int16, 2),
    "I8": (torch.int8, np.int8, 1),
    "U8": (torch.uint8, np.uint8, 1),
    "BOOL": (torch.bool, np.bool_, 1),
}
_NAME_OF = {v[0]: k for k, v in _DTYPES.items()}


class CheckpointError(ValueError):
    """A checkpoint file is malformed or does not hold what the model needs."""


class _Shard:
    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise CheckpointError(f"{path}: too short to be a safetensors file ({size} bytes)")
        self._file = open(path, "rb")
        (hlen,) = struct.unpack("<Q", self._file.read(8))
        if hlen > MAX_HEADER_BYTES or 8 + hlen > size:
            raise CheckpointError(f"{path}: header length {hlen} is past the end of the file or over 256 MiB")
        try:
            header = json.loads(self._file.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise CheckpointError(f"{path}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise CheckpointError(f"{path}: header is not a JSON object")
        self.data_start = 8 + hlen
        data_bytes = size - self.data_start
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            try:
                dtype, shape, (begin, end) = meta["dtype"], tuple(int(s) for s in meta["shape"]), meta["data_offsets"]
            except (KeyError, TypeError, ValueError):
                raise CheckpointError(f"{path}: entry {name!r} lacks dtype, shape or data_offsets") from None
            if dtype not in _DTYPES:
                raise CheckpointError(f"{path}: tensor {name!r} has unknown dtype {dtype!r}")
            if not (0 <= begin <= end <= data_bytes):
                raise CheckpointError(
                    f"{path}: tensor {name!r} spans bytes [{begin}, {end}) but the file holds {data_bytes}")
            want = int(np.prod(shape, dtype=np.int64)) * _DTYPES[dtype][2] if shape else _DTYPES[dtype][2]
            if end - begin != want:
                raise CheckpointError(
                    f"{path}: tensor {name!r} of dtype {dtype} and shape {list(shape)} needs {want} bytes, "
                    f"its byte range holds {end - begin}")
            self.entries[name] = (dtype, shape, begin, end)

    def tensor(self, name: str) -> torch.Tensor:
        dtype, shape, begin, end = self.entries[name]
        tdtype, ndtype, _ = _DTYPES[dtype]
        count = int(np.prod(shape, dtype=np.int64)) if shape else 1
        start = self.data_start + begin
        if start % np.dtype(ndtype).itemsize:
            # a writer that does not align its data: copy this tensor out
            arr = np.frombuffer(bytes(self._map[start:start + (end - begin)]), dtype=ndtype, count=count)
        else:
            arr = np.frombuffer(self._map, dtype=ndtype, count=count, offset=start)
        # the map is read-only; torch only warns about that, and nothing writes through this view
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            t = torch.from_numpy(arr)
        if tdtype is torch.bfloat16:
            t = t.view(torch.bfloat16)
        return t.reshape(shape)


class Checkpoint:
    """All tensors of a model folder, by name."""

    def __init__(self, shards: List[_Shard]):
        self._where: Dict[str, _Shard] = {}
        for s in shards:
            for name in s.entries:
                if name in self._where:
                    raise CheckpointError(f"tensor {name!r} appears in both {self._where[name].path} and {s.path}")
                self._where[name] = s

    @classmethod
    def open(cls, model_dir: str) -> "Checkpoint":
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        if os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as f:
                try:
                    files = sorted(set(json.load(f)["weight_map"].values()))
                except (json.JSONDecodeError, KeyError, AttributeError, TypeError) as e:
                    raise CheckpointError(f"{index}: no usable weight_map: {e}") from None
            shards = []
            for name in files:
                path = os.path.join(model_dir, name)
                if not os.path.isfile(path):
                    raise CheckpointError(f"{index} names shard {name!r}, which is missing")
                shards.append(_Shard(path))
            return cls(shards)
        if os.path.isfile(single):
            return cls([_Shard(single)])
        raise CheckpointError(f"{model_dir}: neither model.safetensors nor model.safetensors.index.json")

    def names(self) -> Iterable[str]:
        return self._where.keys()

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._where[name].entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self._where[name].entries[name][0]][0]

    def get(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise CheckpointError(f"tensor {name!r} not found among {len(self._where)} tensors")
        return self._where[name].tensor(name)


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor]) -> None:
    """Write CPU tensors to one safetensors file, names sorted, data 8-byte aligned."""
    header = {}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAME_OF:
            raise CheckpointError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAME_OF[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().contiguous().cpu()
            if t.dtype is torch.bfloat16:
                t = t.view(torch.int16)
            elif t.dtype is torch.bool:
                t = t.view(torch.uint8)
            f.write(t.numpy().tobytes())
