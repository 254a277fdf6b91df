"""How many pages the cache pool gets: the reference's vectors (tests/unit/kv_autosize_test.cc:14-78)."""
import pytest

from inferx_amd.engine.engine import resolve_kv_blocks

GIB = 1 << 30
MIB = 1 << 20


def test_explicit_blocks_win():
    # kv_autosize_test.cc:14-22: bytes that would be far too small are ignored, and so is a missing page size
    assert resolve_kv_blocks(MIB, explicit_blocks=1234, kv_cache_memory_bytes=1) == 1234
    assert resolve_kv_blocks(0, explicit_blocks=7) == 7


def test_explicit_bytes_beat_utilization():
    # kv_autosize_test.cc:24-32
    got = resolve_kv_blocks(MIB, kv_cache_memory_bytes=4 * GIB, gpu_memory_utilization=0.01, total_bytes=80 * GIB,
                            used_bytes=79 * GIB)
    assert got == 4096


def test_utilization_budget_arithmetic():
    # kv_autosize_test.cc:34-43: 0.5 * 80 GiB - 10 GiB in use - 1 GiB of headroom = 29 GiB of 1 MiB pages
    got = resolve_kv_blocks(MIB, gpu_memory_utilization=0.5, total_bytes=80 * GIB, used_bytes=10 * GIB,
                            headroom_bytes=GIB)
    assert got == 29 * 1024


def test_default_headroom_is_one_gib():
    assert resolve_kv_blocks(MIB, gpu_memory_utilization=0.5, total_bytes=80 * GIB, used_bytes=10 * GIB) == 29 * 1024


def test_too_small_budget_says_what_to_change():
    # kv_autosize_test.cc:45-56: 8 GiB - 7 GiB - 1 GiB = nothing
    with pytest.raises(ValueError, match="raise --gpu-memory-utilization"):
        resolve_kv_blocks(MIB, gpu_memory_utilization=0.1, total_bytes=80 * GIB, used_bytes=7 * GIB,
                          min_blocks=4096)


def test_explicit_bytes_too_small_says_what_to_change():
    # kv_autosize_test.cc:58-67
    with pytest.raises(ValueError, match="--kv-cache-memory-bytes"):
        resolve_kv_blocks(MIB, kv_cache_memory_bytes=MIB, min_blocks=128)


def test_missing_page_bytes_is_an_error():
    # kv_autosize_test.cc:69-72
    with pytest.raises(ValueError):
        resolve_kv_blocks(0, total_bytes=GIB, used_bytes=0)


@pytest.mark.parametrize("bad", [0.0, -0.1, 1.5])
def test_utilization_out_of_range(bad):
    with pytest.raises(ValueError, match="within"):
        resolve_kv_blocks(MIB, gpu_memory_utilization=bad, total_bytes=GIB)
