"""Attention on contexts of 8k to 32k keys against float64 attention: every kernel alone with the numbers of key
slices that the step's plan really picks at such lengths (up to 64), and `PagedAttention.attend` on the steps that
long prompts and long decoding are made of.  The reference's own attention stops at about 12k keys
(src/backends/cuda/ops/layers.cu:256-407, :920-931); this one must not."""
import pytest
import torch

import attention_util as au

pytestmark = pytest.mark.gpu
DEV = au.DEV
TOL = 1.5e-2  # bfloat16 inputs and probabilities, of the largest value (the kernels' tolerance at every length)


def tiles_for(q_lens, tile):
    rows, at = [], 0
    for s, n in enumerate(q_lens):
        rows += [(s, at + q0, min(tile, n - q0)) for q0 in range(0, n, tile)]
        at += n
    return torch.tensor(rows, dtype=torch.int32).t().contiguous().to(DEV)


ONE_TOKEN_CASES = [
    # heads, kv_heads, window, contexts
    (16, 16, 0, [8192, 16384, 32768]),
    (16, 16, 0, [32768]),                      # one request: the plan cuts its keys into 64 slices
    (28, 4, 0, [32768, 8192, 16384, 20001]),   # grouped query heads
    (28, 4, 0, [32767]),
    (16, 16, 4096, [32768, 8192, 5000, 4096]),  # a window of 4,096
    (28, 4, 4096, [30000, 16385]),
]


@pytest.mark.parametrize("heads,kv_heads,window,seq_lens", ONE_TOKEN_CASES)
def test_one_token_steps_on_long_contexts(heads, kv_heads, window, seq_lens):
    """The wavefront-level kernel as a decoding step calls it (loads ahead, grouped heads where heads share keys),
    with the slices of the step's plan and with the most it ever takes."""
    from inferx_amd import ops
    from inferx_amd.parts import attention
    d, page = 128, 16
    q_lens = [1] * len(seq_lens)
    p = au.paged_on_device(seq_lens, q_lens, heads, kv_heads, d, page, seed=len(seq_lens) + heads)
    want = au.reference_for(p, seq_lens, q_lens, d ** -0.5, window)
    grouped = attention.serves_group_together(heads, kv_heads)
    units = len(seq_lens) * (kv_heads if grouped else heads)
    planned = attention._n_splits(units, max(seq_lens), window, 16)
    assert planned >= 16, f"the plan cuts {max(seq_lens)} keys into {planned} slices only"
    for n_splits in sorted({planned, 64, 1}):
        out = torch.full_like(p["q"], float("nan"))
        work = torch.full((len(seq_lens) * heads * n_splits * (d + 2),), float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for(q_lens, 1 if grouped else 16),
                           p["positions"], out, n_splits, work if n_splits > 1 else None, d ** -0.5, window, 16,
                           prefetch=True, grouped=grouped)
        err = au.rel_err(out, want)
        assert err < TOL, f"{n_splits} slices: {err:.3e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_plain_kernel_on_32k_keys(dtype):
    """The kernel of the float32 path (any type): one token and a portion's end on 32,768 keys, a window beside."""
    from inferx_amd import ops
    heads, kv_heads, d, page = 6, 2, 64, 16
    seq_lens, q_lens = [32768, 20000], [1, 5]
    p = au.paged_on_device(seq_lens, q_lens, heads, kv_heads, d, page, seed=3)
    for window in (0, 4096):
        want = au.reference_for(p, seq_lens, q_lens, d ** -0.5, window)
        q, kc, vc = p["q"].to(dtype), p["k_cache"].to(dtype), p["v_cache"].to(dtype)
        out = torch.full_like(q, float("nan"))
        ops.attention_plain(q, kc, vc, p["table"], p["seq_of_token"], p["positions"], out, d ** -0.5, window)
        err = au.rel_err(out, want)
        assert err < (1e-5 if dtype == torch.float32 else TOL), f"window {window}: {err:.3e}"


def _plant(p, s, row, far, gain):
    """Key `far` of request s becomes `gain` times the query of row `row` (all key/value heads: the mean of the
    query heads that share each), so that this key's score stands far above all others."""
    k, v = p["dense"][s]
    q = p["qs"][s][row].float()
    kv_heads = k.shape[1]
    k[far] = (q.view(kv_heads, -1, q.shape[-1]).mean(1) * gain).to(k.dtype)
    au.write_request(p, s)
    return v[far]


@pytest.mark.parametrize("far", [0, 17, 511, 512, 16383, 16384, 32751, 32767])
def test_one_far_key_among_32k_decoding(far):
    """One key of 32,768 matches the query: the output is that key's value, whichever slice, page or end of the
    context it lies in (the wavefront-level kernel, heads alone and grouped, 64 and the planned number of slices;
    the plain kernel)."""
    from inferx_amd import ops
    L, d, page = 32768, 128, 16
    for heads, kv_heads, grouped in ((4, 4, False), (8, 2, True)):
        p = au.paged_on_device([L], [1], heads, kv_heads, d, page, seed=far % 97)
        if grouped:  # the heads of a group ask the same question
            p["qs"][0][:] = p["qs"][0].view(1, kv_heads, -1, d)[:, :, :1].expand(1, kv_heads, heads // kv_heads, d) \
                .reshape(1, heads, d)
            p["q"] = p["qs"][0].clone()
        value = _plant(p, 0, 0, far, 3.0)
        want = value.repeat_interleave(heads // kv_heads, 0).float()
        for n_splits in (64, 16, 1):
            out = torch.full_like(p["q"], float("nan"))
            work = torch.empty(heads * n_splits * (d + 2), dtype=torch.float32, device=DEV)
            ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for([1], 1 if grouped else 16),
                               p["positions"], out, n_splits, work if n_splits > 1 else None, d ** -0.5, 0, 16,
                               prefetch=True, grouped=grouped)
            assert float((out[0].float() - want).abs().max()) < 0.02 * float(want.abs().max()), \
                f"key {far}, {n_splits} slices, grouped={grouped}"
        out = torch.full_like(p["q"], float("nan"))
        ops.attention_plain(p["q"], p["k_cache"], p["v_cache"], p["table"], p["seq_of_token"], p["positions"], out,
                            d ** -0.5, 0)
        assert float((out[0].float() - want).abs().max()) < 0.02 * float(want.abs().max()), f"plain, key {far}"


@pytest.mark.parametrize("tile", [64, 128])
def test_far_keys_among_32k_for_a_portion(tile):
    """A portion of 256 queries on top of 32,512 keys through the LDS-sharing kernels, its keys in 1, 8 and 64
    slices: a few queries each match one key far before them, at slice and page edges and at the context's ends."""
    from inferx_amd import ops
    L, n, d, heads, page = 32768, 256, 128, 2, 16
    p = au.paged_on_device([L], [n], heads, heads, d, page, seed=21)
    pairs = [(0, 0), (1, 32512), (63, 4095), (64, 4096), (100, 16383), (128, 16384), (200, 32511), (255, 32767),
             (254, 20000)]  # (query row, key); a key at or before the row's own position
    values = {}
    for row, far in pairs:
        assert far <= L - n + row
        values[row] = _plant(p, 0, row, far, 3.0).float()
    want = au.reference_for(p, [L], [n], d ** -0.5, 0)
    tiles = tiles_for([n], tile)
    for slices in (1, 8, 64):
        out = torch.full_like(p["q"], float("nan"))
        work = torch.full((n * heads * slices * (d + 2),), float("nan"), dtype=torch.float32, device=DEV)
        ops.attention_prefill(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles, p["positions"], out, d ** -0.5, 0,
                              tile, None, slices, work if slices > 1 else None)
        assert au.rel_err(out, want) < TOL, f"{slices} slices"
        for row, _ in pairs:
            assert float((out[row].float() - values[row]).abs().max()) < 0.02 * float(values[row].abs().max()), \
                f"row {row}, {slices} slices"


STEP_CASES = [
    # heads, kv, head size, window, q_lens, seq_lens, what the plan must choose
    (16, 16, 128, 0, [1, 1, 1], [8192, 16384, 32768], "one token each, 32 slices"),
    (16, 16, 128, 0, [1], [32768], "one token each, 64 slices"),
    (28, 4, 128, 0, [1, 1, 1, 1], [32768, 8192, 16384, 20001], "grouped, 64 slices"),
    (28, 4, 128, 4096, [1, 1], [30000, 16385], "grouped, 32 slices"),
    (16, 16, 128, 4096, [1, 1, 1], [32768, 8192, 5000], "one token each, 32 slices"),
    (16, 16, 128, 0, [2048], [30000], "portion in tiles"),
    (16, 16, 128, 0, [512], [30000], "portion in slices"),
    (16, 16, 112, 0, [2048], [30000], "portion in slices"),    # (tiles of 64 queries: no tiles of 128 for this head)
    (28, 4, 128, 0, [2048], [32048], "portion in tiles"),
    (28, 4, 128, 0, [200], [32048], "portion in slices"),
    (16, 16, 128, 0, [2048] * 8, [30000, 2048, 9000, 30000, 16000, 30000, 22000, 30000], "portion in tiles"),
    (16, 16, 80, 0, [2048] * 4, [30000, 2048, 9000, 16000], "portions in pairs"),
    (28, 4, 128, 0, [1] * 32 + [512, 512], [4096] * 32 + [4096, 8192], "portions beside grouped tokens"),
    (16, 16, 128, 4096, [2048, 1], [20000, 30000], "portion and a token, window"),
]


@pytest.mark.parametrize("heads,kv,d,window,q_lens,seq_lens,expect", STEP_CASES)
def test_steps_on_long_contexts_through_the_part(heads, kv, d, window, q_lens, seq_lens, expect):
    """`PagedAttention.attend` on the steps that long prompts and long decoding consist of, pages from the cache
    manager: whichever kernels and slice counts the step's plan picks, the result is float64 attention."""
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import CacheBinding, Runtime
    from inferx_amd.parts import attention, build_part
    from test_gpu_parts import make_ctx
    rt = Runtime("bfloat16")
    page = 16
    part = build_part("mixer", PartSpec("attention", {"hidden_size": 64, "num_heads": heads, "num_kv_heads": kv,
                                                      "head_dim": d, "window": window}))
    pages = sum(-(-L // page) for L in seq_lens) + 2
    ctx, batch = make_ctx(rt, q_lens, seq_lens, page, pages)
    p = au.paged_on_device(seq_lens, q_lens, heads, kv, d, page, seed=5, table=batch.block_tables[0], pages=pages)
    want = au.reference_for(p, seq_lens, q_lens, d ** -0.5, window)
    out = torch.full_like(p["q"], float("nan"))
    part.attend(ctx, p["q"], CacheBinding(group=0, arrays=dict(k=p["k_cache"], v=p["v_cache"])), out)
    err = au.rel_err(out, want)
    assert err < TOL, f"{expect}: {err:.3e}"
    if expect.startswith(("one token each", "grouped")):
        _, _, n_splits, grouped = attention.query_tiles(ctx, window, heads, d, kv)
        assert grouped == expect.startswith("grouped") and f"{n_splits} slices" in expect, (n_splits, grouped)
    else:
        tile = attention.WIDE_PREFILL_TILE if d % 32 == 0 else attention.PREFILL_TILE
        lds, waves = attention.mixed_step_plan(ctx, window, heads, kv, True, tile)
        if expect == "portion in slices":
            assert lds[2] > 1 and not waves
        elif expect == "portion in tiles":
            assert lds[2] == 1 and int(lds[1][1].max()) < 0 and not waves
        elif expect == "portions in pairs":
            assert lds[2] == 1 and int(lds[1][1].max()) >= 0 and not waves
        elif expect == "portions beside grouped tokens":
            assert lds is not None and len(waves) == 1 and waves[0][4]
        else:
            assert lds is not None and len(waves) == 1
