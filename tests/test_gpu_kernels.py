"""Each kernel alone against a plain float32/float64 PyTorch reference of the same
operation, at sizes other than the engine's tiny configurations."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, tol, what=""):
    want = want.double().cpu()
    err = float((got.double().cpu() - want).abs().max()) / max(float(want.abs().max()), 1e-30)
    assert err <= tol, f"{what}: error {err:.3e} of the largest value, tolerance {tol:.1e}"
    return err


TOL = {torch.float32: 1e-5, torch.bfloat16: 1.5e-2}


# ---------------------------------------------------------------------------
def build_paged(seq_lens, q_lens, heads, kv_heads, d, page_size, dtype, seed=0, shuffle_pages=True):
    """Random q/k/v for requests of the given context and query lengths, written into a paged cache whose pages
    are handed out in a scrambled order.  Returns everything the attention kernels need plus dense k, v."""
    from inferx_amd import ops  # noqa: F401
    S = len(seq_lens)
    max_blocks = max(-(-L // page_size) for L in seq_lens) + 1
    total_pages = sum(-(-L // page_size) for L in seq_lens) + 3
    order = torch.randperm(total_pages, generator=torch.Generator().manual_seed(seed)).tolist() if shuffle_pages \
        else list(range(total_pages))
    table = torch.full((S, max_blocks), -1, dtype=torch.int32)
    k_cache = torch.zeros(total_pages, kv_heads, page_size, d, dtype=dtype)
    v_cache = torch.zeros(total_pages, kv_heads, d, page_size, dtype=dtype)
    dense, qs, positions, seq_of_token = [], [], [], []
    nxt = 0
    for s, (L, n) in enumerate(zip(seq_lens, q_lens)):
        k = (torch.randn(L, kv_heads, d, generator=torch.Generator().manual_seed(seed * 100 + s))).to(dtype)
        v = (torch.randn(L, kv_heads, d, generator=torch.Generator().manual_seed(seed * 100 + s + 50))).to(dtype)
        dense.append((k, v))
        for j in range(-(-L // page_size)):
            page = order[nxt]
            nxt += 1
            table[s, j] = page
            chunk = slice(j * page_size, min(L, (j + 1) * page_size))
            m = chunk.stop - chunk.start
            k_cache[page, :, :m, :] = k[chunk].transpose(0, 1)
            v_cache[page, :, :, :m] = v[chunk].permute(1, 2, 0)
        qs.append(torch.randn(n, heads, d, generator=torch.Generator().manual_seed(seed * 100 + s + 77)).to(dtype))
        positions += list(range(L - n, L))
        seq_of_token += [s] * n
    return dict(q=torch.cat(qs).to(DEV), k_cache=k_cache.to(DEV), v_cache=v_cache.to(DEV), table=table.to(DEV),
                positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
                seq_of_token=torch.tensor(seq_of_token, dtype=torch.int32, device=DEV), dense=dense, qs=qs)


def attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window):
    outs = []
    for (k, v), q, L, n in zip(p["dense"], p["qs"], seq_lens, q_lens):
        q, k, v = q.double(), k.double(), v.double()
        kk, vv = k.repeat_interleave(heads // kv_heads, 1), v.repeat_interleave(heads // kv_heads, 1)
        s = torch.einsum("qhd,khd->hqk", q, kk) * scale
        qpos = torch.arange(L - n, L)[:, None]
        kpos = torch.arange(L)[None, :]
        ok = kpos <= qpos
        if window > 0:
            ok &= kpos >= qpos + 1 - window
        s = s.masked_fill(~ok[None], -math.inf)
        outs.append(torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), vv))
    return torch.cat(outs)


ATTN_CASES = [
    # seq_lens, q_lens, heads, kv_heads, d, page, window
    ([40], [40], 4, 2, 32, 16, 0),
    ([300, 5, 129], [300, 5, 129], 6, 2, 48, 16, 0),
    ([700, 33, 1], [1, 1, 1], 8, 8, 128, 16, 0),          # decoding, long context: keys are split
    ([513, 260], [2, 17], 4, 1, 64, 32, 0),               # portions on top of a context
    ([400, 90, 31], [400, 1, 31], 3, 3, 16, 16, 24),      # window
    ([1000, 999], [1, 3], 2, 1, 80, 64, 100),             # window, decoding, big pages
    ([2100], [1], 16, 16, 128, 16, 0),
]


@pytest.mark.parametrize("case", ATTN_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_plain(case, dtype):
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = case
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, dtype, seed=3)
    out = torch.empty_like(p["q"])
    scale = d ** -0.5
    ops.attention_plain(p["q"], p["k_cache"], p["v_cache"], p["table"], p["seq_of_token"], p["positions"], out, scale,
                        window)
    close(out, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), TOL[dtype], "attention_plain")


def tiles_for(q_lens, tile=16):
    rows, at = [], 0
    for s, n in enumerate(q_lens):
        for q0 in range(0, n, tile):
            rows.append((s, at + q0, min(tile, n - q0)))
        at += n
    return torch.tensor(rows, dtype=torch.int32).t().contiguous().to(DEV)


@pytest.mark.parametrize("tile", [16, 32, -16])  # -16: tiles of 16 with prefetch
@pytest.mark.parametrize("n_splits", [1, 3, 8, 70])
@pytest.mark.parametrize("case", ATTN_CASES)
def test_attention_mfma(case, n_splits, tile):
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = case
    prefetch, tile = tile < 0, abs(tile)
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=4)
    out = torch.full_like(p["q"], float("nan"))
    T = p["q"].shape[0]
    work = torch.empty(T * heads * n_splits * (d + 2), dtype=torch.float32, device=DEV) if n_splits > 1 else None
    scale = d ** -0.5
    ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for(q_lens, tile), p["positions"], out,
                       n_splits, work, scale, window, tile, prefetch)
    close(out, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), TOL[torch.bfloat16],
          f"attention_mfma splits={n_splits} tile={tile}")


GROUPED_CASES = [
    # seq_lens, q_lens, heads, kv_heads, d, page, window
    ([700, 33, 1], [1, 1, 1], 28, 4, 128, 16, 0),         # seven query heads per key/value head
    ([1000, 999, 64], [1, 3, 2], 32, 2, 80, 64, 100),     # sixteen; window; requests of two and three tokens
    ([130, 17], [1, 1], 6, 3, 48, 16, 0),                 # two
    ([257], [1], 8, 2, 256, 32, 40),
]


@pytest.mark.parametrize("prefetch", [False, True])
@pytest.mark.parametrize("n_splits", [1, 3, 8, 70])
@pytest.mark.parametrize("case", GROUPED_CASES)
def test_attention_mfma_grouped_queries(case, n_splits, prefetch):
    """One token per tile, the query heads of a key/value head side by side in it."""
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = case
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=6)
    out = torch.full_like(p["q"], float("nan"))
    T = p["q"].shape[0]
    work = torch.empty(T * heads * n_splits * (d + 2), dtype=torch.float32, device=DEV) if n_splits > 1 else None
    scale = d ** -0.5
    ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for(q_lens, 1), p["positions"], out,
                       n_splits, work, scale, window, 16, prefetch, grouped=True)
    close(out, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), TOL[torch.bfloat16],
          f"attention_mfma grouped splits={n_splits}")


PREFILL_CASES = ATTN_CASES + [
    ([1500], [1500], 5, 1, 128, 16, 0),                   # many tiles of one request
    ([777, 300], [130, 300], 4, 2, 112, 16, 0),           # a portion that starts off a tile's edge; odd head blocks
    ([900, 450], [500, 450], 2, 2, 96, 32, 70),           # window shorter than a workgroup's queries
]


def outside_in_pairs(n_tiles):
    """Tile i with tile n - 1 - i (the middle one alone): two tiles per workgroup, of different requests and lengths."""
    half = (n_tiles + 1) // 2
    second = [n_tiles - 1 - i if n_tiles - 1 - i >= half else -1 for i in range(half)]
    return torch.tensor([list(range(half)), second], dtype=torch.int32).to(DEV)


PREFILL128_CASES = [c for c in PREFILL_CASES if c[4] % 32 == 0] + [
    ([1500, 64], [1500, 3], 3, 1, 32, 16, 0),
    ([2100, 300], [900, 300], 4, 2, 96, 64, 0),           # three 32s of the head; pages of 64
    ([700, 450], [690, 450], 2, 2, 64, 32, 200),          # a window that passes rounds within a tile
]


def prefill_cases(tile):
    return PREFILL_CASES if tile == 64 else PREFILL128_CASES


@pytest.mark.parametrize("paired", [False, True])
@pytest.mark.parametrize("tile,index", [(64, i) for i in range(len(PREFILL_CASES))] +
                         [(128, i) for i in range(len(PREFILL128_CASES))])
def test_attention_prefill(tile, index, paired):
    """The kernels whose wavefronts share keys through LDS (tiles of 64 queries, 16 per wavefront; tiles of 128, 32
    per wavefront, with wavefronts that only load), against float64 attention per request."""
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = prefill_cases(tile)[index]
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=6)
    out = torch.full_like(p["q"], float("nan"))
    scale = d ** -0.5
    tiles = tiles_for(q_lens, tile)
    ops.attention_prefill(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles, p["positions"],
                          out, scale, window, tile, outside_in_pairs(tiles.shape[1]) if paired else None)
    close(out, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), TOL[torch.bfloat16],
          f"attention_prefill tile={tile}")


@pytest.mark.parametrize("paired", [False, True])
@pytest.mark.parametrize("n_splits", [2, 3, 16])
@pytest.mark.parametrize("tile,index", [(64, i) for i in range(len(PREFILL_CASES))] +
                         [(128, i) for i in range(len(PREFILL128_CASES))])
def test_attention_prefill_with_key_slices(tile, index, n_splits, paired):
    """Every tile's keys cut into slices, a workgroup per slice (or two slices), parts put together afterwards:
    with more slices than a tile has rounds of keys some are empty."""
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = prefill_cases(tile)[index]
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=7)
    out = torch.full_like(p["q"], float("nan"))
    T = p["q"].shape[0]
    scale = d ** -0.5
    tiles = tiles_for(q_lens, tile)
    work = torch.full((T * heads * n_splits * (d + 2),), float("nan"), dtype=torch.float32, device=DEV)
    ops.attention_prefill(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles, p["positions"], out, scale, window,
                          tile, outside_in_pairs(tiles.shape[1] * n_splits) if paired else None, n_splits, work)
    close(out, attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window), TOL[torch.bfloat16],
          f"attention_prefill slices={n_splits}")


@pytest.mark.parametrize("tile", [64, 128])
def test_attention_prefill_finds_far_keys(tile):
    """Each of a few queries of a long portion matches one key far before it: its output must be that key's value
    (a tile staged from the wrong page, a wrong causal bound of a wavefront or a stale LDS buffer would miss)."""
    from inferx_amd import ops
    L, n, d, heads = 1200, 500, 64, 2
    p = build_paged([L], [n], heads, heads, d, 16, torch.bfloat16, seed=9)
    k, v = p["dense"][0]
    q = p["qs"][0]
    pairs = [(0, 0), (63, 640), (64, 63), (130, 829), (257, 700), (499, 1199), (300, 1000)]  # (query row, key)
    for row, far in pairs:
        assert far <= L - n + row
        page, off = int(p["table"][0, far // 16]), far % 16
        p["k_cache"][page, :, off, :] = (q[row] * 6.0).to(DEV)
        k[far] = q[row] * 6.0
    out = torch.empty_like(p["q"])
    ops.attention_prefill(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for([n], tile), p["positions"], out,
                          d ** -0.5, 0, tile)
    close(out, attention_reference(p, [L], [n], heads, heads, d ** -0.5, 0), TOL[torch.bfloat16], "far keys")
    for row, far in pairs:
        assert float((out[row].float().cpu() - v[far].float()).abs().max()) < 0.05 * float(v[far].abs().max())


def test_attention_finds_one_far_key():
    """One key among 2,000 matches the query: the output must be that key's value (a skipped page, a wrong
    split boundary or a wrong table entry would miss it)."""
    from inferx_amd import ops
    L, d, heads = 2000, 64, 2
    for far in (0, 15, 16, 777, 1024, 1999):
        p = build_paged([L], [1], heads, heads, d, 16, torch.bfloat16, seed=far)
        k, v = p["dense"][0]
        q = p["qs"][0]
        # rewrite the far key in the cache so that q . k is large there
        page, off = int(p["table"][0, far // 16]), far % 16
        p["k_cache"][page, :, off, :] = (q[0] * 4.0).to(DEV)
        k[far] = q[0] * 4.0
        for n_splits in (1, 5):
            out = torch.empty_like(p["q"])
            work = torch.empty(heads * n_splits * (d + 2), dtype=torch.float32, device=DEV)
            ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for([1]), p["positions"], out,
                               n_splits, work, d ** -0.5, 0)
            want = attention_reference(p, [L], [1], heads, heads, d ** -0.5, 0)
            close(out, want, TOL[torch.bfloat16], f"far key {far}")
            assert float((out[0].float().cpu() - v[far].float()).abs().max()) < 0.05 * float(v[far].abs().max())


def poison_what_no_query_may_read(p, seq_lens, q_lens, page_size, window):
    """Everything in the pool that the requests do not own becomes NaN, as an earlier request that went wrong
    might have left it: unused pages, the part of each request's last page past its last token, page 0 (which is
    freed for it and read as a filler), and, with a window, the pages that all of a request's queries have passed,
    whose table entries become -1 as the cache manager leaves them."""
    table = p["table"].cpu().clone()
    k_cache, v_cache = p["k_cache"], p["v_cache"]
    pages = k_cache.shape[0]
    used = set(int(x) for x in table.flatten() if x >= 0)
    spare = [i for i in range(pages) if i not in used]
    if 0 in used:  # move page 0's content elsewhere so that page 0 is nobody's
        to = spare.pop()
        k_cache[to], v_cache[to] = k_cache[0].clone(), v_cache[0].clone()
        table[table == 0] = to
    nan = float("nan")
    for s, (L, n) in enumerate(zip(seq_lens, q_lens)):
        last = (L - 1) // page_size
        tail = L - last * page_size
        pg = int(table[s, last])
        k_cache[pg, :, tail:, :] = nan
        v_cache[pg, :, :, tail:] = nan
        if window > 0:
            first_read = max(0, (L - n) + 1 - window)  # the lowest key that the request's first query reads
            for j in range(first_read // page_size):
                pg = int(table[s, j])
                k_cache[pg], v_cache[pg] = nan, nan
                table[s, j] = -1
    owned = set(int(x) for x in table.flatten() if x >= 0)
    for i in range(pages):
        if i not in owned:
            k_cache[i], v_cache[i] = nan, nan
    p["table"] = table.to(DEV)


NAN_CASES = [
    # seq_lens, q_lens, heads, kv_heads, d, page, window
    ([700, 33, 1], [1, 1, 1], 8, 8, 128, 16, 0),
    ([1000, 999, 70], [1, 3, 2], 8, 2, 64, 64, 100),       # window: passed pages are -1 and hold NaN
    ([513, 260, 45], [200, 17, 45], 4, 1, 64, 32, 0),      # portions whose last page is partly filled
    ([900, 450], [500, 450], 2, 2, 96, 32, 70),
]


@pytest.mark.parametrize("case", NAN_CASES)
def test_attention_kernels_ignore_what_other_requests_left_in_the_pool(case):
    """A request that once wrote NaN into its keys or values leaves them in its freed pages.  Whoever gets such a
    page, or reads page 0 as a filler for a page the window has passed, must not be touched by them: a masked
    key's probability is zero, and zero times NaN is NaN unless the value is masked too."""
    from inferx_amd import ops
    seq_lens, q_lens, heads, kv_heads, d, page, window = case
    scale = d ** -0.5
    p = build_paged(seq_lens, q_lens, heads, kv_heads, d, page, torch.bfloat16, seed=12)
    want = attention_reference(p, seq_lens, q_lens, heads, kv_heads, scale, window)
    poison_what_no_query_may_read(p, seq_lens, q_lens, page, window)
    T = p["q"].shape[0]
    runs = []
    for n_splits in (1, 4):
        work = torch.empty(T * heads * n_splits * (d + 2), dtype=torch.float32, device=DEV)
        for prefetch in (False, True):
            out = torch.full_like(p["q"], float("nan"))
            ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for(q_lens), p["positions"], out,
                               n_splits, work, scale, window, 16, prefetch)
            runs.append((f"wavefront-level, {n_splits} slices, prefetch {prefetch}", out))
        if max(q_lens) < heads // kv_heads or all(n == 1 for n in q_lens):
            out = torch.full_like(p["q"], float("nan"))
            ops.attention_mfma(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles_for(q_lens, 1), p["positions"],
                               out, n_splits, work, scale, window, 16, True, grouped=heads > kv_heads)
            runs.append((f"one token per tile, {n_splits} slices", out))
        for tile in (64, 128):
            out = torch.full_like(p["q"], float("nan"))
            tiles = tiles_for(q_lens, tile)
            ops.attention_prefill(p["q"], p["k_cache"], p["v_cache"], p["table"], tiles, p["positions"], out, scale,
                                  window, tile, None, n_splits, work if n_splits > 1 else None)
            runs.append((f"LDS-sharing, tiles of {tile}, {n_splits} slices", out))
    out = torch.full_like(p["q"], float("nan"))
    ops.attention_plain(p["q"], p["k_cache"], p["v_cache"], p["table"], p["seq_of_token"], p["positions"], out, scale,
                        window)
    runs.append(("plain", out))
    for what, out in runs:
        assert torch.isfinite(out.float()).all(), f"{what}: NaN from the pool reached the output"
        close(out, want, TOL[torch.bfloat16], what)
