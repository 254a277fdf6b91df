"""Causal attention over the paged cache, grouped-query, with optional bias on
q/k/v, an optional window and a pluggable position encoding.

One fused product gives q|k|v (rows of the three weights stacked, reference
src/model/qwen2.cc:1368-1403); one kernel adds the bias, rotates q and k and
appends k, v to the cache (:920-969); attention reads keys [start, p] through
the request's block table (layers.cu:256-318, window :329-407); then the output
product (:1026-1027).
"""
from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch

from .. import ops
from ..config.spec import PartSpec
from .base import CacheNeed, Mixer, ParamSpec, build_part, register_part
from .dense_mlp import stack_rows


class PagedAttention(Mixer):
    graph_safe = True  # the query tiles are planned on the host, but outside a captured step (see capture_plan)

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, qkv_bias: bool = True,
                 out_bias: bool = False, window: int = 0, scale: Optional[float] = None,
                 position: Optional[PartSpec] = None, init_std: float = 0.02):
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head_dim {head_dim} must be even and at most 256")
        self.out_bias = bool(out_bias)
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.qkv_bias, self.window = int(head_dim), bool(qkv_bias), int(window)
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5
        self.init_std = float(init_std)
        self.position = build_part("position", position) if position is not None else None
        # the part of every head that the position encoding rotates: (first element, number of elements)
        self.rotated = (0, self.head_dim)
        if self.position is not None:
            self.rotated = (int(getattr(self.position, "begin", 0)), int(getattr(self.position, "rotary_dim", self.head_dim)))
            begin, dim = self.rotated
            if begin < 0 or dim <= 0 or dim % 2 or begin + dim > self.head_dim:
                raise ValueError(f"the position encoding rotates elements {begin} to {begin + dim} of heads of "
                                 f"{self.head_dim}: an even number of elements within the head is needed")
        self.w_qkv = self.b_qkv = self.w_out = self.b_out = None

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    def cache_need(self) -> CacheNeed:
        return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, self.window)

    def subparts(self):
        return [self.position]

    def param_specs(self) -> List[ParamSpec]:
        H, s = self.hidden_size, self.init_std
        specs = [ParamSpec("q_proj.weight", (self.q_dim, H), std=s), ParamSpec("k_proj.weight", (self.kv_dim, H), std=s),
                 ParamSpec("v_proj.weight", (self.kv_dim, H), std=s), ParamSpec("o_proj.weight", (H, self.q_dim), std=s)]
        if self.qkv_bias:
            specs += [ParamSpec("q_proj.bias", (self.q_dim,), std=s), ParamSpec("k_proj.bias", (self.kv_dim,), std=s),
                      ParamSpec("v_proj.bias", (self.kv_dim,), std=s)]
        if self.out_bias:
            specs.append(ParamSpec("o_proj.bias", (H,), std=s))
        return specs

    def bind(self, tensors, rt) -> None:
        self.w_qkv = stack_rows([tensors[f"{n}_proj.weight"] for n in "qkv"])
        self.b_qkv = stack_rows([tensors[f"{n}_proj.bias"] for n in "qkv"]) if self.qkv_bias else None
        self.w_out = tensors["o_proj.weight"].contiguous()
        self.b_out = tensors["o_proj.bias"].contiguous() if self.out_bias else None
        if self.position is not None:
            self.position.bind({}, rt)

    def capture_plan(self, ctx, requests: int, longest: int) -> None:
        """The query tiles of a step of one token per request never change: tile i = request i, row i, one query;
        the slices of the keys follow from `longest`."""
        key = ("attention_tiles_host", QUERY_TILE)
        if key not in ctx.memo:
            tiles = torch.tensor([list(range(requests)), list(range(requests)), [1] * requests], dtype=torch.int32,
                                 device=ctx.rt.device)
            ctx.memo[key] = (tiles, requests, longest)

    def forward(self, ctx, x, cache):
        rt = ctx.rt
        T = x.shape[0]
        table = self.position.prepare(ctx) if self.position is not None else None
        q = rt.empty((T, self.num_heads, self.head_dim))
        writes = cache.writes
        epilogue = (self.b_qkv, table, ctx.slots[cache.group] if writes else None, q, cache.k if writes else None,
                    cache.v if writes else None, self.num_heads, self.num_kv_heads, self.head_dim)
        whole = table is None or self.rotated == (0, self.head_dim)
        if (T <= 32 and x.dtype == torch.bfloat16 and self.w_qkv.dtype == torch.bfloat16 and self.head_dim % 32 == 0
                and self.hidden_size % 8 == 0 and whole):
            ops.qkv_rope_skinny(x, self.w_qkv, *epilogue)  # few tokens: product and epilogue in one launch
        else:
            ops.qkv_rope_append(rt.linear(x, self.w_qkv), *epilogue, rotated=None if whole else self.rotated)
        out = rt.empty((T, self.num_heads, self.head_dim))
        self.attend(ctx, q, cache, out)
        y = rt.linear(out.view(T, self.q_dim), self.w_out)
        if self.b_out is not None:
            ops.add_bias(y, self.b_out)
        return y

    def attend(self, ctx, q, cache, out) -> None:
        """bfloat16 with pages and heads in multiples of 16: the matrix-core kernels (the one that shares keys through
        LDS for the prompt portions of a step, the wavefront-level one for requests that bring few tokens and for
        steps of one token per request); else the plain one."""
        page_size = cache.k.shape[2]
        if q.dtype == torch.bfloat16 and page_size % 16 == 0 and self.head_dim % 16 == 0:
            T = ctx.num_tokens
            if not ctx.one_token_each:  # some request brings more than one token: the step's plan says who goes where
                lds_fits = self.head_dim <= 128 and page_size & (page_size - 1) == 0
                tile = WIDE_PREFILL_TILE if self.head_dim % 32 == 0 else PREFILL_TILE
                lds, waves = mixed_step_plan(ctx, self.window, self.num_heads, self.num_kv_heads, lds_fits, tile)
                table = ctx.block_tables[cache.group]
                if lds is not None:
                    tiles, pairs, slices = lds
                    work = None
                    if slices > 1:
                        work = ctx.rt.empty((T * self.num_heads * slices * (self.head_dim + 2),), torch.float32)
                    ops.attention_prefill(q, cache.k, cache.v, table, tiles, ctx.positions, out, self.scale,
                                          self.window, tile, pairs, slices, work)
                for rows, tiles, positions, n_splits, grouped in waves:
                    # a launch that serves some of the step's requests gets their rows put side by side
                    qs = q if rows is None else q.index_select(0, rows)
                    outs = out if rows is None else torch.empty_like(qs)
                    work = None
                    if n_splits > 1:
                        work = ctx.rt.empty((qs.shape[0] * self.num_heads * n_splits * (self.head_dim + 2),),
                                            torch.float32)
                    ops.attention_mfma(qs, cache.k, cache.v, table, tiles, positions, outs, n_splits, work,
                                       self.scale, self.window, QUERY_TILE, grouped=grouped)
                    if rows is not None:
                        out.index_copy_(0, rows, outs)
                return
            tiles, tile, n_splits, grouped = query_tiles(ctx, self.window, self.num_heads, self.head_dim,
                                                         self.num_kv_heads)
            work = None
            if n_splits > 1:
                work = ctx.rt.empty((q.shape[0] * self.num_heads * n_splits * (self.head_dim + 2),), torch.float32)
            ops.attention_mfma(q, cache.k, cache.v, ctx.block_tables[cache.group], tiles, ctx.positions, out,
                               n_splits, work, self.scale, self.window, tile, prefetch=True, grouped=grouped)
        else:
            ops.attention_plain(q, cache.k, cache.v, ctx.block_tables[cache.group], ctx.seq_of_token, ctx.positions,
                                out, self.scale, self.window)


# ---- the wavefront-level kernel (ops.attention_mfma)
QUERY_TILE = 16          # queries of one request per wavefront ...
LARGE_QUERY_TILE = 32    # ... or 32 when the step brings many tokens (keys and values are then read once per 32)
LARGE_TILE_TOKENS = 1 << 30  # measured: no faster than tiles of 16 on MI355X, so off
WAVES_WANTED = 2048      # two wavefronts per SIMD of 256 compute units: measured best at batch 8 (longer slices per wavefront)
MIN_KEYS_PER_SPLIT = 128
# ---- the LDS-sharing kernel (ops.attention_prefill) takes the requests of a step that bring at least
# PREFILL_MIN_ROWS tokens each, if they bring PREFILL_MIN_TOKENS together and make enough workgroups: at least
# PREFILL_MIN_WORKGROUPS (tile, head) pairs, or a context of PREFILL_SLICED_MIN_ROUNDS rounds of 64 keys, which
# is then cut into slices of at least PREFILL_SLICE_ROUNDS rounds (see mixed_step_plan)
PREFILL_TILE = 64        # queries of one request per workgroup ...
# ... or 128 where the head size is a multiple of 32: 32 queries per wavefront, wavefronts of their own for the loads,
# and the key slices chosen by another rule (see mixed_step_plan).  Measured against tiles of 64 at their best, heads
# of 128: 2,048 tokens of 16 heads 48 against 62 us, 8,192 tokens 343 against 562, 2,048 tokens of 28 heads on 30,000
# keys 1,118 against 1,675, 256 tokens on 8,192 keys 39 against 51, 64 tokens on 2,048 keys 22 against 23.
WIDE_PREFILL_TILE = 128
PREFILL_MIN_ROWS = 16
PREFILL_MIN_TOKENS = 128
PREFILL_MIN_WORKGROUPS = 120
PREFILL_SLICED_MIN_ROUNDS = 96
PREFILL_SLICE_ROUNDS = 8


def plan_tiles(ctx, tile: int):
    """Tiles of up to `tile` consecutive queries per request (int32 [3, n]: request, first row, rows) on the
    device, their number, and the longest context.  Planned on the host from the step's batch, once per step; a
    captured step finds its (static) plan already in `ctx.memo`."""
    base = ctx.memo.get(("attention_tiles_host", tile))
    if base is None:
        b = ctx.host
        n = (b.q_start[1:] - b.q_start[:-1]).astype(np.int64)
        tiles_host = _tiles_of(n, b.q_start[:-1].astype(np.int64), np.arange(len(n)), tile)
        tiles_dev = torch.from_numpy(np.ascontiguousarray(tiles_host)).to(ctx.rt.device)
        longest = int(b.seq_lens.max()) if len(b.seq_lens) else 0
        base = ctx.memo[("attention_tiles_host", tile)] = (tiles_dev, tiles_host.shape[1], longest)
    return base


def _tiles_of(n: np.ndarray, first_row: np.ndarray, seqs: np.ndarray, tile: int) -> np.ndarray:
    """Tiles of up to `tile` consecutive rows for the requests `seqs` (n: their new tokens, first_row: where their
    rows start): int32 [3, tiles] = request, first row, rows."""
    counts = -(-n // tile)
    which = np.repeat(np.arange(len(n)), counts)
    first = np.cumsum(counts) - counts
    off = (np.arange(int(counts.sum())) - np.repeat(first, counts)) * tile
    rows = np.minimum(tile, n[which] - off)
    return np.stack([seqs[which], first_row[which] + off, rows]).astype(np.int32)


def _pairs_by_work(t: np.ndarray, b, window: int, pair: bool, slices: int = 1) -> np.ndarray:
    """Which two tiles each workgroup of the LDS-sharing kernel takes, int32 [2, n_pairs].  A tile's work grows
    with the keys it reads (all up to its last query, or a window of them), so the tile that reads most is paired
    with the one that reads least, and so on inwards: workgroups then take about equally long.  Pairs are ordered
    by falling work.  Without `pair` every tile gets a workgroup of its own, the ones that read most first; with
    `slices` > 1 every slice of every tile does (unit = tile * slices + slice)."""
    t = t.astype(np.int64)
    n_tiles = t.shape[1]
    new = (b.q_start[1:] - b.q_start[:-1]).astype(np.int64)
    first_row = t[1] - b.q_start[:-1].astype(np.int64)[t[0]]           # the tile's first query within its portion
    end = b.seq_lens.astype(np.int64)[t[0]] - new[t[0]] + first_row + t[2]  # one past the last key it reads
    start = np.maximum(0, end - t[2] + 1 - window) if window > 0 else np.zeros_like(end)
    work = -(-(end - (start // 64) * 64) // 64)  # rounds of 64 keys
    order = np.argsort(-work, kind="stable")
    half = (n_tiles + 1) // 2
    if slices > 1:
        pairs = np.full((2, n_tiles * slices), -1, dtype=np.int32)
        pairs[0] = (order[:, None] * slices + np.arange(slices)[None, :]).ravel()
        return pairs
    if not pair:
        pairs = np.full((2, n_tiles), -1, dtype=np.int32)
        pairs[0] = order
        return pairs
    pairs = np.full((2, half), -1, dtype=np.int32)
    pairs[0] = order[:half]
    pairs[1, :n_tiles - half] = order[::-1][:n_tiles - half]
    return pairs


def serves_group_together(heads: int, kv_heads: int) -> bool:
    """Whether a one-token tile of the wavefront-level kernel holds the query heads of a key/value head (2 to 16 of
    them) side by side, so that its keys and values are read once for all of them."""
    return 2 <= heads // kv_heads <= 16


def mixed_step_plan(ctx, window: int, heads: int, kv_heads: int, lds_fits: bool = True, tile: int = PREFILL_TILE):
    """Who serves which requests of a step in which some request brings more than one token: (lds, waves).

    lds = (tiles, pairs, slices) for the LDS-sharing kernel, rows as in the step, or None.  It takes the requests
    that bring at least PREFILL_MIN_ROWS tokens, in tiles of `tile` queries (64 or 128), if they bring
    PREFILL_MIN_TOKENS together and make enough workgroups (below); slices: into how many workgroups each tile's
    keys are cut.

    waves = launches of the wavefront-level kernel for the other requests, each (rows, tiles, positions, slices of
    the keys, grouped): where query heads share key/value heads, requests that bring fewer tokens than a key/value
    head has query heads -- the decoding requests of a mixed step -- are served a token per tile with those heads
    side by side (`grouped`), the rest in tiles of QUERY_TILE queries of one head.  `rows` are the launch's rows in
    the step, to be put side by side for it, or None if it is the step's only launch and takes all rows as they lie.

    Sent through the LDS-sharing kernel, a decoding request would walk its whole context alone, with one query of
    a tile's 64 at work and once per query head (measured at 32 decoding requests with 4,096 keys beside two
    portions of 512, 28 query heads on 4: 487 us per layer; 162 + 57 us in two launches)."""
    key = ("attention_mixed", window, heads, kv_heads, lds_fits, tile)
    if key in ctx.memo:
        return ctx.memo[key]
    b = ctx.host
    dev = ctx.rt.device
    q_start = b.q_start[:-1].astype(np.int64)
    n = (b.q_start[1:] - b.q_start[:-1]).astype(np.int64)
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    long = n >= PREFILL_MIN_ROWS
    seqs = np.flatnonzero(long)
    t = _tiles_of(n[seqs], q_start[seqs], seqs, tile) if (lds_fits and len(seqs)) else None
    # The LDS-sharing kernel walks a tile's keys in one workgroup.  With few tiles that leaves compute units idle
    # however long the context is (128 queries of 16 heads on 30,000 keys: 638 us in 32 workgroups).  Then, from
    # about 6,000 keys on, every tile's keys are cut into slices with a workgroup each, about a thousand in all and
    # none under eight rounds of 64 keys (97 us in the example; the wavefront-level kernel, which also cuts keys
    # into slices, 152 us).  On shorter contexts the slices' parts cost more than they gain (a floor of about
    # 45 us), and the wavefront-level kernel takes steps of fewer than PREFILL_MIN_WORKGROUPS (tile, head) pairs
    # (2,048 keys + 128 queries: 24 against 52 us); from there on the LDS-sharing kernel is level or ahead.
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    slices = 1
    wide = tile == WIDE_PREFILL_TILE
    if t is not None and wide:
        # Tiles of 128 queries: a workgroup fills a compute unit, so what counts is a workgroup per compute unit.
        # With fewer (tile, head) pairs than that, the keys are cut into as many slices as make them up, none under
        # eight rounds of 64 keys, 32 at most (64 tokens of 16 heads on 8,192 keys: 25 us in 16 slices against 141
        # in one; 1,024 tokens of 28 heads on 30,000 keys, 224 pairs: one slice is best).
        keys = int(b.seq_lens[seqs].max())
        rounds = -(-(min(keys, window + tile) if window > 0 else keys) // 64)
        slices = max(1, min(cus // (t.shape[1] * heads), rounds // PREFILL_SLICE_ROUNDS, 32))
        slices = 1 << (slices.bit_length() - 1)
    elif t is not None and t.shape[1] * heads < 8 * cus:
        keys = int(b.seq_lens[seqs].max())
        rounds = -(-(min(keys, window + PREFILL_TILE) if window > 0 else keys) // 64)
        if rounds >= PREFILL_SLICED_MIN_ROUNDS:
            # (with two to eight workgroups per compute unit a few slices still even out what the compute units
            # get: 2,048 queries of 28 heads on 30,000 keys, 896 workgroups, 1.53 against 1.73 ms in four slices)
            want = (4 if t.shape[1] * heads < 2 * cus else 16) * cus
            slices = max(1, min(want // (t.shape[1] * heads), rounds // PREFILL_SLICE_ROUNDS, 64))
            slices = 1 << (slices.bit_length() - 1)
    lds = None
    served = np.zeros(len(n), dtype=bool)
    if t is not None and int(n[long].sum()) >= PREFILL_MIN_TOKENS and \
            (wide or slices > 1 or t.shape[1] * heads >= PREFILL_MIN_WORKGROUPS):
        # Two workgroups fit a compute unit.  Pairs only when that still leaves two per compute unit: with fewer,
        # a workgroup per tile keeps two wavefronts on a SIMD instead of one (measured: two portions of 512 on 28
        # heads, 448 tiles, 15.2 against 15.8 ms for a step of 8 layers; 2,048 tokens on 16 heads, 512 tiles, 15.5
        # against 15.4 ms for 24 layers).
        # (tiles of 128 queries are never paired: the workgroups are started in the order of falling work, and one
        # fills a compute unit)
        pairs = _pairs_by_work(t, b, window, pair=not wide and slices == 1 and t.shape[1] * heads >= 2 * cus,
                               slices=slices)
        lds = (to_dev(t), to_dev(pairs), slices)
        served = long.copy()
    group = heads // kv_heads
    together = serves_group_together(heads, kv_heads)
    sets = [(~served & (n > 0) & (n < group), True), (~served & (n >= group), False)] if together \
        else [(~served & (n > 0), False)]
    sets = [(np.flatnonzero(mask), grouped) for mask, grouped in sets if mask.any()]
    waves = []
    for seqs, grouped in sets:
        ns = n[seqs]
        alone = lds is None and len(sets) == 1
        first = q_start[seqs] if alone else np.cumsum(ns) - ns
        st = _tiles_of(ns, first, seqs, 1 if grouped else QUERY_TILE)
        rows = positions = None
        if alone:
            positions = ctx.positions
        else:
            rows = to_dev(np.concatenate([np.arange(q_start[i], q_start[i] + n[i]) for i in seqs]))
            positions = ctx.positions.index_select(0, rows)
        units = st.shape[1] * (kv_heads if grouped else heads)
        waves.append((rows, to_dev(st), positions, _n_splits(units, int(b.seq_lens[seqs].max()), window, QUERY_TILE),
                      grouped))
    ctx.memo[key] = (lds, waves)
    return ctx.memo[key]


def _n_splits(units: int, longest: int, window: int, tile: int) -> int:
    """Into how many slices the wavefront-level kernel cuts each tile's keys: enough for WAVES_WANTED wavefronts,
    no slice shorter than MIN_KEYS_PER_SPLIT, a power of two (few distinct values, few captured graphs)."""
    span = min(longest, window + tile + 32) if window > 0 else longest
    n_splits = 1 if units >= 2048 else max(1, min(WAVES_WANTED // max(1, units), -(-span // MIN_KEYS_PER_SPLIT), 64))
    return 1 << (n_splits.bit_length() - 1)


def query_tiles(ctx, window: int, heads: int, head_dim: int = 128, kv_heads: Optional[int] = None):
    """The wavefront-level kernel's plan: tiles (see plan_tiles), the tile size (16 or 32), into how many
    slices each tile's keys are cut, and whether a tile is one token with its grouped query heads (a step in which
    every request brings one token, and query heads share key/value heads)."""
    tile = LARGE_QUERY_TILE if (ctx.num_tokens >= LARGE_TILE_TOKENS and head_dim <= 128) else QUERY_TILE
    kv_heads = kv_heads or heads
    key = ("attention_tiles", window, heads, kv_heads, tile)
    hit = ctx.memo.get(key)
    if hit is not None:
        return hit
    tiles_dev, n_tiles, longest = plan_tiles(ctx, tile)
    grouped = tile == QUERY_TILE and ctx.one_token_each and serves_group_together(heads, kv_heads)
    units = n_tiles * (kv_heads if grouped else heads)
    ctx.memo[key] = (tiles_dev, tile, _n_splits(units, longest, window, tile), grouped)
    return ctx.memo[key]


register_part("mixer", "attention", PagedAttention)
