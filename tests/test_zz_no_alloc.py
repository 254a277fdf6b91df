"""`ix_attention_mfma_noalloc`, the attention entry point that takes its slices' partial results to a buffer
inside the library instead of a workspace of the caller's: called through ctypes, twice in a row (the second
call smaller, so that it finds the first call's leftovers in the buffer), and compared bit for bit with
`ix_attention_mfma` on a workspace, which runs the same kernels."""
import ctypes

import pytest
import torch

from test_gpu_kernels import DEV, attention_reference, build_paged, close, tiles_for

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 16 << 20  # IX_ATTENTION_SCRATCH_BYTES of inferx_amd/csrc/inferx_hip.h


def _p(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _run(lib, p, tiles, out, n_splits, heads, kv_heads, d, page, window, scale, workspace=None, grouped=False):
    """Through the entry point with a workspace if one is given, else through the one that allocates nothing."""
    T = p["q"].shape[0]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = [_p(p["q"]), _p(p["k_cache"]), _p(p["v_cache"]), _p(p["table"]), _p(tiles[0]), _p(tiles[1]), _p(tiles[2]),
            _p(p["positions"]), _p(out)]
    tail = [ctypes.c_int64(T), ctypes.c_int(tiles.shape[1]), ctypes.c_int(16), ctypes.c_int(n_splits),
            ctypes.c_int(heads), ctypes.c_int(kv_heads), ctypes.c_int(d), ctypes.c_int(page),
            ctypes.c_int(p["table"].shape[1]), ctypes.c_float(scale), ctypes.c_int(window), ctypes.c_int(1),
            ctypes.c_int(1 if grouped else 0), stream]
    if workspace is not None:
        parts = T * heads * n_splits
        ws = [_p(workspace), ctypes.c_void_p(workspace.data_ptr() + 4 * parts * d)]
        return lib.ix_attention_mfma(*head, *ws, *tail)
    return lib.ix_attention_mfma_noalloc(*head, *tail)


CALLS = [
    # seq_lens, q_lens, heads, kv_heads, d, page, window, n_splits: a big call, then a smaller one
    (([1500, 700, 33, 1200], [1, 1, 1, 1], 16, 16, 128, 16, 0, 8), ([300, 90], [1, 1], 16, 16, 128, 16, 0, 2)),
    (([900, 410, 77], [5, 1, 17], 8, 2, 64, 32, 0, 4), ([130], [3], 8, 2, 64, 32, 64, 2)),
]


@pytest.mark.parametrize("calls", CALLS)
def test_no_alloc_entry_point_equals_the_one_with_a_workspace(calls):
    from inferx_amd import ops
    lib = ops.lib()
    for i, (seq_lens, q_lens, heads, kv_heads, d, page, window, n_splits) in enumerate(calls):
        p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=11 + i)
        tiles = tiles_for(q_lens)
        T, scale = p["q"].shape[0], d ** -0.5
        want, got = torch.empty_like(p["q"]), torch.full_like(p["q"], float("nan"))
        workspace = torch.empty(T * heads * n_splits * (d + 2), dtype=torch.float32, device=DEV)
        assert _run(lib, p, tiles, want, n_splits, heads, kv_heads, d, page, window, scale, workspace) == 0
        if i == 0:  # (the first call on a device looks the array's address up; it allocates nothing either)
            assert _run(lib, p, tiles, got, n_splits, heads, kv_heads, d, page, window, scale) == 0
        # what the driver says is free on the device: an allocation by the library itself, which the tensor
        # library's own counters would not see, shows here
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        rc = _run(lib, p, tiles, got, n_splits, heads, kv_heads, d, page, window, scale)
        assert rc == 0, lib.ix_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was taken during the call"
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"call {i} differs from the workspace one"
        close(got, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), 1.5e-2, f"call {i}")


def test_no_alloc_entry_point_without_slices_and_grouped():
    from inferx_amd import ops
    lib = ops.lib()
    seq_lens, q_lens, heads, kv_heads, d, page = [640, 200, 31], [1, 1, 1], 12, 3, 128, 16
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=5)
    tiles = tiles_for(q_lens, tile=1)
    scale = d ** -0.5
    ref = attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, 0)
    for n_splits in (4, 1):
        got = torch.full_like(p["q"], float("nan"))
        rc = _run(lib, p, tiles, got, n_splits, heads, kv_heads, d, page, 0, scale, grouped=True)
        assert rc == 0, lib.ix_last_error().decode()
        close(got, ref, 1.5e-2, f"grouped, {n_splits} slices")


def test_no_alloc_entry_point_refuses_what_does_not_fit():
    from inferx_amd import ops
    lib = ops.lib()
    heads, d, n_splits = 16, 128, 64
    tokens = SCRATCH_BYTES // 4 // (heads * n_splits * (d + 2)) + 1  # one token too many
    seq_lens, q_lens = [tokens + 40], [tokens]
    p = build_paged(seq_lens, q_lens, heads, heads, d, 16, torch.bfloat16, seed=2)
    tiles = tiles_for(q_lens)
    out = torch.zeros_like(p["q"])
    assert _run(lib, p, tiles, out, n_splits, heads, heads, d, 16, 0, d ** -0.5) == 1
    msg = lib.ix_last_error().decode()
    assert "do not fit" in msg and str(SCRATCH_BYTES) in msg
    torch.cuda.synchronize()
    assert not out.any()  # nothing ran
    # the largest that fits runs
    p = build_paged([tokens + 39], [tokens - 1], heads, heads, d, 16, torch.bfloat16, seed=2)
    tiles = tiles_for([tokens - 1])
    out = torch.empty_like(p["q"])
    assert _run(lib, p, tiles, out, n_splits, heads, heads, d, 16, 0, d ** -0.5) == 0
    close(out, attention_reference(p, [tokens + 39], [tokens - 1], heads, heads, d ** -0.5, 0), 1.5e-2, "largest")
