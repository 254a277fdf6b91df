"""Weights by name, their errors, and the random-weights mode (no GPU).
Error cases follow the reference's tests/unit/safetensors_test.cc:173-251."""
import json
import os
import struct

import pytest
import torch

from inferx_amd.config import config_from_dict
from inferx_amd.parts import build_model
from inferx_amd.weights import (Checkpoint, CheckpointError, check_names_and_shapes, random_tensors,
                                write_model_folder, write_safetensors)
import tiny


def test_random_folder_round_trip(tmp_path):
    cfg = config_from_dict(tiny.CONFIG_B)
    write_model_folder(cfg, 5, str(tmp_path), "bfloat16")
    ck = Checkpoint.open(str(tmp_path))
    model = build_model(cfg.model_spec())
    expected = model.expected_tensors()
    assert set(ck.names()) == set(expected)
    assert "lm_head.weight" not in expected  # tied
    for name, p in expected.items():
        t = ck.get(name)
        assert tuple(t.shape) == tuple(p.shape) and t.dtype == torch.bfloat16
    # the library's reader sees the same bytes as ours
    from safetensors.torch import load_file
    theirs = load_file(os.path.join(str(tmp_path), "model.safetensors"))
    for name in expected:
        assert torch.equal(theirs[name], ck.get(name))
    assert float(ck.get("model.norm.weight").float().min()) == 1.0
    w = ck.get("model.layers.1.mlp.experts.3.up_proj.weight").float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    with open(os.path.join(str(tmp_path), "config.json")) as f:
        assert config_from_dict(json.load(f)).num_experts == 8


def test_reads_what_the_library_writes(tmp_path):
    from safetensors.torch import save_file
    tensors = {"a": torch.arange(6, dtype=torch.float32).view(2, 3), "b": torch.ones(5, dtype=torch.bfloat16),
               "c": torch.arange(4, dtype=torch.int32)}
    save_file(tensors, os.path.join(str(tmp_path), "model.safetensors"))
    ck = Checkpoint.open(str(tmp_path))
    for k, v in tensors.items():
        assert torch.equal(ck.get(k), v) and ck.dtype(k) == v.dtype


def test_seed_and_dtype(tmp_path):
    cfg = config_from_dict(tiny.CONFIG_A)
    model = build_model(cfg.model_spec())
    a, b, c = random_tensors(model, 1, "float32"), random_tensors(model, 1, "bfloat16"), random_tensors(model, 2, "float32")
    name = "model.layers.0.self_attn.q_proj.weight"
    assert torch.equal(a[name].to(torch.bfloat16), b[name])  # one draw, two roundings
    assert not torch.equal(a[name], c[name])
    assert a["model.layers.0.self_attn.q_proj.bias"].abs().max() > 0


def test_a_random_value_depends_on_seed_name_and_index_alone():
    """The generator is counter-based: element i of a tensor is a function of (seed, name, i), whatever the
    tensor's shape or the other tensors; 64-bit integer arithmetic reference for the first elements."""
    from inferx_amd.weights.random_init import counter_normal
    a = counter_normal(7, "model.layers.3.mlp.gate.weight", (60, 2048), 0.02)
    assert torch.equal(a.flatten()[:1000], counter_normal(7, "model.layers.3.mlp.gate.weight", (1000,), 0.02))
    assert not torch.equal(a, counter_normal(7, "model.layers.4.mlp.gate.weight", (60, 2048), 0.02))
    assert not torch.equal(a, counter_normal(8, "model.layers.3.mlp.gate.weight", (60, 2048), 0.02))
    big = counter_normal(1, "w", (1 << 20,), 1.0)
    assert abs(float(big.mean())) < 5e-3 and abs(float(big.std()) - 1.0) < 5e-3
    assert 0.001 < float((big.abs() > 3).float().mean()) < 0.004  # the tails of a normal distribution, nearly
    # the same numbers from plain Python integers (no tensor library in the way)
    import zlib
    mask = (1 << 64) - 1

    def mix(z):
        z &= mask
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
        return z ^ (z >> 31)
    key = mix(mix(1) ^ (zlib.crc32(b"w") * 0x9E3779B97F4A7C15))
    for i in (0, 1, 2, 77, (1 << 20) - 1):
        total = 0
        for j in range(3):
            h = mix((3 * i + j) * 0x9E3779B97F4A7C15 + key)
            total += sum((h >> s) & 0xFFFF for s in (0, 16, 32, 48))
        assert float(big[i]) == (total - 393210) / 65536.0


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(tiny.CONFIG_A)
    model = build_model(cfg.model_spec())
    tensors = random_tensors(model, 1, "bfloat16")
    del tensors["model.layers.1.mlp.gate.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.mlp.extra.weight"] = torch.zeros(3, dtype=torch.bfloat16)
    tensors["lm_head.weight"] = torch.zeros(255, 64, dtype=torch.bfloat16)
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), tensors)
    expected = {n: tuple(p.shape) for n, p in model.expected_tensors().items()}
    with pytest.raises(CheckpointError) as e:
        check_names_and_shapes(expected, Checkpoint.open(str(tmp_path)))
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.1.mlp.gate.weight" in msg and "model.norm.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.0.mlp.extra.weight" in msg
    assert "wrong shapes (1)" in msg and "lm_head.weight: expected [256, 64], file has [255, 64]" in msg


def _write_raw(path, header: dict, data: bytes, header_len=None):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob) if header_len is None else header_len))
        f.write(blob)
        f.write(data)


@pytest.mark.parametrize("header, data, header_len, needle", [
    ({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 16]}}, b"\0" * 8, None, "file holds"),
    ({"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8, None, "needs 12 bytes"),
    ({"t": {"dtype": "Q7", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 8, None, "unknown dtype"),
    ({"t": {"dtype": "F32", "shape": [2]}}, b"\0" * 8, None, "lacks dtype, shape or data_offsets"),
    ({}, b"", 1 << 40, "header length"),
])
def test_malformed_files(tmp_path, header, data, header_len, needle):
    _write_raw(os.path.join(str(tmp_path), "model.safetensors"), header, data, header_len)
    with pytest.raises(CheckpointError) as e:
        Checkpoint.open(str(tmp_path))
    assert needle in str(e.value)


def test_missing_tensor_and_missing_file(tmp_path):
    with pytest.raises(CheckpointError):
        Checkpoint.open(str(tmp_path))
    write_safetensors(os.path.join(str(tmp_path), "model.safetensors"), {"a": torch.zeros(2)})
    with pytest.raises(CheckpointError) as e:
        Checkpoint.open(str(tmp_path)).get("b")
    assert "'b' not found among 1 tensors" in str(e.value)


def test_sharded(tmp_path):
    d = str(tmp_path)
    write_safetensors(os.path.join(d, "s1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(os.path.join(d, "s2.safetensors"), {"b": torch.zeros(3)})
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}, f)
    ck = Checkpoint.open(d)
    assert sorted(ck.names()) == ["a", "b"] and ck.shape("b") == (3,)
    os.remove(os.path.join(d, "s2.safetensors"))
    with pytest.raises(CheckpointError) as e:
        Checkpoint.open(d)
    assert "missing" in str(e.value)
    write_safetensors(os.path.join(d, "s2.safetensors"), {"a": torch.zeros(3)})
    with pytest.raises(CheckpointError) as e:
        Checkpoint.open(d)
    assert "appears in both" in str(e.value)


def test_tensors_are_fetched_when_asked_for_and_not_kept():
    """The mapping that `load_weights` returns brings a tensor in when the model's `bind` asks for it and keeps
    only what more than one part claims."""
    from inferx_amd.weights.loader import LazyWeights
    fetched = []

    def fetch(name):
        fetched.append(name)
        return torch.full((2,), float(len(fetched)))

    w = LazyWeights(["a", "b", "tied"], fetch, shared=["tied"])
    assert list(w) == ["a", "b", "tied"] and len(w) == 3 and "a" in w and "c" not in w
    first, again = w["a"], w["a"]
    assert fetched == ["a", "a"] and first is not again           # nothing is kept
    t1, t2 = w["tied"], w["tied"]
    assert fetched == ["a", "a", "tied"] and t1 is t2             # what two parts claim is fetched once
    with pytest.raises(KeyError):
        w["c"]
    w.clear()
    assert len(w) == 0 and "a" not in w
    with pytest.raises(KeyError):
        w["a"]
