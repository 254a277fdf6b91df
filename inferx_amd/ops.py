"""Python face of the HIP library: one function per kernel entry point.

Each function checks on the host what its kernel assumes (device, dtype,
contiguity, shapes, index ranges where cheap), passes raw device pointers and
the current HIP stream, and raises `KernelError` with the library's message when
a launch is refused.  There is no fallback: without a GPU and the built library
these functions fail.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from .csrc import build as _build

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def lib():
    return _build.load()


def _dt(t: torch.Tensor) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not float32 or bfloat16") from None


# The entry points' argument types are set when the library is loaded (csrc/build.py `signatures`), so the
# helpers below hand over plain Python values: an address or None for a pointer, ints and floats for numbers.
def _ptr(t: Optional[torch.Tensor]):
    if t is None:
        return None
    if t.is_contiguous() and t.is_cuda:
        return t.data_ptr()
    raise KernelError("kernel operands must live on the GPU (no CPU path exists)" if not t.is_cuda
                      else "kernel operands must be contiguous")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current HIP stream of the current device (what torch launches on, also under graph capture)."""
    if _raw_stream is not None and _raw_device is not None:
        # the same value as below, without building a Stream object (17 us a call) or the checks of
        # torch.cuda.current_device (1 us)
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


_i64 = int
_i32 = int
_f32 = float
_functions = {}


def _call(name: str, *args):
    fn = _functions.get(name)
    if fn is None:
        fn = _functions[name] = getattr(lib(), name)
    if fn(*args) != 0:
        raise KernelError(lib().ix_last_error().decode("utf-8", "replace"))


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _is_i32(t, n=None):
    _need(t.dtype == torch.int32, "index arrays must be int32")
    if n is not None:
        _need(t.numel() >= n, f"index array holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------------
def embed(h: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """h[t] = table[ids[t]] * scale; h float32 [T, H]."""
    T, H = h.shape
    _need(h.dtype == torch.float32, "the residual stream is float32")
    _need(table.dim() == 2 and table.shape[1] == H, "table width differs from h")
    _is_i32(ids, T)
    _call("ix_embed", _ptr(h), _ptr(table), _i32(_dt(table)), _ptr(ids), _i64(T), _i64(H), _i64(table.shape[0]),
          _f32(scale), _stream())


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, out: torch.Tensor, eps: float,
                rows: Optional[torch.Tensor] = None) -> None:
    """out = rmsnorm(h + delta) * weight; h += delta in place when `rows` is None.
    With `rows`, out[r] is computed from row rows[r] and h is not changed."""
    H = h.shape[1]
    _need(h.dtype == torch.float32, "the residual stream is float32")
    _need(weight.numel() == H and out.shape[1] == H, "width mismatch")
    n_out = out.shape[0]
    if rows is None:
        _need(n_out == h.shape[0], "out must have a row per row of h")
    else:
        _is_i32(rows, n_out)
    if delta is not None:
        _need(delta.shape == h.shape, "delta must have the shape of h")
    _call("ix_add_rmsnorm", _ptr(h), _ptr(delta), _i32(_dt(delta) if delta is not None else F32), _ptr(weight),
          _i32(_dt(weight)), _ptr(out), _i32(_dt(out)), _ptr(rows), _i64(n_out), _i64(H), _f32(eps), _stream())


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, i] = silu(gate_up[t, i]) * gate_up[t, W + i]."""
    T, W2 = gate_up.shape
    _need(W2 % 2 == 0 and out.shape == (T, W2 // 2) and out.dtype == gate_up.dtype, "shape or dtype mismatch")
    _call("ix_silu_mul", _ptr(gate_up), _ptr(out), _i32(_dt(out)), _i64(T), _i64(W2 // 2), _stream())


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> None:
    """y [T, N] += bias [N], in place (summed in float32, rounded to y's type)."""
    _need(y.dim() == 2 and y.is_contiguous() and bias.numel() == y.shape[1], "bias must hold one number per column")
    _call("ix_add_bias", _ptr(y), _i32(_dt(y)), _ptr(bias), _i32(_dt(bias)), _i64(y.shape[0]), _i64(y.shape[1]),
          _stream())


def rope_table(cos_sin: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> None:
    """cos_sin[t, j] = (cos, sin)(positions[t] * inv_freq[j]); float32 [T, half, 2]."""
    T, half, two = cos_sin.shape
    _need(two == 2 and cos_sin.dtype == torch.float32 and inv_freq.dtype == torch.float32, "float32 tables needed")
    _need(inv_freq.numel() == half, "inv_freq length differs")
    _is_i32(positions, T)
    _call("ix_rope_table", _ptr(cos_sin), _ptr(positions), _ptr(inv_freq), _i64(T), _i32(half), _stream())


def qkv_rope_append(qkv: torch.Tensor, bias: Optional[torch.Tensor], cos_sin: Optional[torch.Tensor],
                    slots: Optional[torch.Tensor], q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                    v_cache: Optional[torch.Tensor], heads: int, kv_heads: int, head_dim: int,
                    rotated: Optional[Tuple[int, int]] = None) -> None:
    """Bias, rotation and cache append after the fused q/k/v product.
    qkv [T, (heads + 2 kv_heads) * d]; key cache [pages, kv_heads, page_size, d], value cache
    [pages, kv_heads, d, page_size].  `rotated` = (first element, number of elements) of every head that the
    table rotates (the whole head if not given); the table is [T, elements / 2, 2]."""
    T = qkv.shape[0]
    rot_begin, rot_dim = rotated if rotated is not None else (0, head_dim)
    _need(0 <= rot_begin and rot_dim >= 0 and rot_dim % 2 == 0 and rot_begin + rot_dim <= head_dim,
          "the rotated part must be an even number of elements within the head")
    width = (heads + 2 * kv_heads) * head_dim
    _need(qkv.shape == (T, width), f"qkv must be [T, {width}]")
    _need(q_out.dtype == qkv.dtype and q_out.numel() == T * heads * head_dim, "q_out mismatch")
    if bias is not None:
        _need(bias.numel() == width, "bias length differs")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.shape == (T, rot_dim // 2, 2), "rotary table mismatch")
    page_size, total = 1, 0
    if k_cache is not None:
        _need(v_cache is not None and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype, "cache mismatch")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == kv_heads and k_cache.shape[3] == head_dim, "cache layout")
        _need(v_cache.shape == (k_cache.shape[0], kv_heads, head_dim, k_cache.shape[2]), "value cache layout")
        page_size = k_cache.shape[2]
        total = k_cache.shape[0] * page_size
        _need(slots is not None, "slots needed to write the cache")
        _is_i32(slots, T)
    _call("ix_qkv_rope_append", _ptr(qkv), _i32(_dt(qkv)), _ptr(bias), _i32(_dt(bias) if bias is not None else F32),
          _ptr(cos_sin), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _i64(T), _i32(heads),
          _i32(kv_heads), _i32(head_dim), _i32(page_size), _i64(total), _i32(rot_begin), _i32(rot_dim), _stream())


def qkv_rope_skinny(x: torch.Tensor, w_qkv: torch.Tensor, bias: Optional[torch.Tensor],
                    cos_sin: Optional[torch.Tensor], slots: Optional[torch.Tensor], q_out: torch.Tensor,
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], heads: int, kv_heads: int,
                    head_dim: int) -> None:
    """For at most 32 tokens (bfloat16): the q/k/v product, bias, rotation and cache append in one launch."""
    T, K = x.shape
    width = (heads + 2 * kv_heads) * head_dim
    _need(x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16 and q_out.dtype == torch.bfloat16,
          "the fused q/k/v kernel is bfloat16 only")
    _need(w_qkv.shape == (width, K), f"q/k/v weight must be [{width}, {K}]")
    _need(q_out.numel() == T * heads * head_dim, "q_out mismatch")
    if bias is not None:
        _need(bias.numel() == width, "bias length differs")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.shape == (T, head_dim // 2, 2), "rotary table mismatch")
    page_size, total = 1, 0
    if k_cache is not None:
        _need(v_cache is not None and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16,
              "cache mismatch")
        _need(k_cache.dim() == 4 and k_cache.shape[1] == kv_heads and k_cache.shape[3] == head_dim, "cache layout")
        _need(v_cache.shape == (k_cache.shape[0], kv_heads, head_dim, k_cache.shape[2]), "value cache layout")
        page_size = k_cache.shape[2]
        total = k_cache.shape[0] * page_size
        _need(slots is not None, "slots needed to write the cache")
        _is_i32(slots, T)
    _call("ix_qkv_rope_skinny", _ptr(x), _ptr(w_qkv), _ptr(bias), _i32(_dt(bias) if bias is not None else F32),
          _ptr(cos_sin), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), _i32(T), _i64(K), _i32(heads),
          _i32(kv_heads), _i32(head_dim), _i32(page_size), _i64(total), _stream())


def _check_caches(q, k_cache, v_cache):
    d = q.shape[2]
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "cache dtype differs from q")
    _need(k_cache.dim() == 4 and k_cache.shape[3] == d, "key cache must be [pages, kv_heads, page_size, d]")
    _need(v_cache.shape == (k_cache.shape[0], k_cache.shape[1], d, k_cache.shape[2]),
          "value cache must be [pages, kv_heads, d, page_size]")


def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                    seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float,
                    window: int) -> None:
    """Paged attention, one workgroup per (token, head).  q, out [T, heads, d]."""
    T, heads, d = q.shape
    _need(out.shape == q.shape and out.dtype == q.dtype, "out mismatch")
    _check_caches(q, k_cache, v_cache)
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(seq_of_token, T)
    _is_i32(positions, T)
    _call("ix_attention_plain", _ptr(q), _ptr(k_cache), _ptr(v_cache), _i32(_dt(q)), _ptr(block_table),
          _ptr(seq_of_token), _ptr(positions), _ptr(out), _i64(T), _i32(heads), _i32(kv_heads), _i32(d),
          _i32(page_size), _i32(block_table.shape[1]), _f32(scale), _i32(window), _stream())


def attention_mfma(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                   tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, n_splits: int,
                   workspace: Optional[torch.Tensor], scale: float, window: int, tile_queries: int = 16,
                   prefetch: bool = False, grouped: bool = False) -> None:
    """Paged attention on the matrix cores (bfloat16).  `tiles` int32 [3, n_tiles]: request, first token row and
    number of rows (<= tile_queries, which is 16 or 32) of each query tile.  `workspace` float32 with T * heads * n_splits * (d + 2) entries
    when n_splits > 1.  `grouped`: every tile is ONE token, and the query heads of a key/value head (at most 16)
    are served together, so that its keys and values are read once for all of them."""
    T, heads, d = q.shape
    _need(q.dtype == torch.bfloat16, "the matrix-core attention kernel is bfloat16 only")
    _need(out.shape == q.shape and out.dtype == q.dtype, "out mismatch")
    _check_caches(q, k_cache, v_cache)
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(positions, T)
    _is_i32(tiles)
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    n_tiles = tiles.shape[1]
    _need(not grouped or (tile_queries == 16 and heads // kv_heads <= 16 and n_tiles <= T),
          "grouped queries: one token per tile, tiles of 16, at most 16 query heads per key/value head")
    part_o = part_ml = None
    if n_splits > 1:
        need = T * heads * n_splits * (d + 2)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"workspace of {need} float32 needed")
        part_o = workspace
        part_ml = workspace[T * heads * n_splits * d:]
    _call("ix_attention_mfma", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
          _ptr(tiles[1]), _ptr(tiles[2]), _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml), _i64(T),
          _i32(n_tiles), _i32(tile_queries), _i32(n_splits), _i32(heads), _i32(kv_heads), _i32(d), _i32(page_size),
          _i32(block_table.shape[1]), _f32(scale), _i32(window), _i32(1 if prefetch else 0),
          _i32(1 if grouped else 0), _stream())


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      tiles: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, scale: float, window: int,
                      tile_queries: int = 64, pairs: Optional[torch.Tensor] = None, n_splits: int = 1,
                      workspace: Optional[torch.Tensor] = None) -> None:
    """Paged attention for prompt portions (bfloat16, head_dim <= 128): tiles of up to 64 queries of one
    request, keys and values shared through LDS; or, with `tile_queries` 128 (head_dim a multiple of 32), tiles of
    up to 128 queries, 32 per wavefront, with wavefronts of their own for the loads.  `tiles` as for attention_mfma.  `pairs` int32 [2, n]: the two
    units that workgroup i takes one after the other (second -1: none); every unit is to be named exactly once
    (a tile left out stays unwritten).  Without `pairs` every unit gets a workgroup of its own.

    A unit is a tile, or with n_splits > 1 slice `unit % n_splits` of the keys of tile `unit // n_splits`; then
    `workspace` (float32, T * heads * n_splits * (d + 2) entries) takes the slices' parts, and ALL T rows of `out`
    are written from it: rows that no tile covers get no meaningful values and are for the caller to fill."""
    T, heads, d = q.shape
    _need(q.dtype == torch.bfloat16, "the matrix-core attention kernel is bfloat16 only")
    _need(out.shape == q.shape and out.dtype == q.dtype, "out mismatch")
    _check_caches(q, k_cache, v_cache)
    kv_heads, page_size = k_cache.shape[1], k_cache.shape[2]
    _need(block_table.dim() == 2, "block table must be [requests, pages]")
    _is_i32(block_table)
    _is_i32(positions, T)
    _is_i32(tiles)
    _need(tiles.dim() == 2 and tiles.shape[0] == 3 and tiles.is_contiguous(), "tiles must be int32 [3, n_tiles]")
    n_units = tiles.shape[1] * n_splits
    if pairs is None:
        pairs = torch.stack([torch.arange(n_units, dtype=torch.int32), torch.full((n_units,), -1, dtype=torch.int32)])
        pairs = pairs.to(q.device)
    _is_i32(pairs)
    _need(pairs.dim() == 2 and pairs.shape[0] == 2 and pairs.is_contiguous(), "pairs must be int32 [2, n_pairs]")
    _need(pairs.shape[1] <= n_units <= 2 * pairs.shape[1], "pairs must name every unit once")
    _need(page_size & (page_size - 1) == 0, "this kernel takes pages of a power of two of keys")
    part_o = part_ml = None
    if n_splits > 1:
        need = T * heads * n_splits * (d + 2)
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              f"workspace of {need} float32 needed")
        part_o = workspace
        part_ml = workspace[T * heads * n_splits * d:]
    if tile_queries == 128:
        _need(d % 32 == 0, "tiles of 128 queries take head sizes in steps of 32")
        _call("ix_attention_prefill128", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
              _ptr(tiles[1]), _ptr(tiles[2]), _ptr(pairs[0]), _ptr(pairs[1]), _i32(pairs.shape[1]), _ptr(positions),
              _ptr(out), _ptr(part_o), _ptr(part_ml), _i32(n_splits), _i64(T), _i32(tiles.shape[1]), _i32(heads),
              _i32(kv_heads), _i32(d), _i32(page_size), _i32(block_table.shape[1]), _f32(scale), _i32(window),
              _stream())
        return
    _call("ix_attention_prefill", _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _ptr(tiles[0]),
          _ptr(tiles[1]), _ptr(tiles[2]), _ptr(pairs[0]), _ptr(pairs[1]), _i32(pairs.shape[1]), _ptr(positions),
          _ptr(out), _ptr(part_o), _ptr(part_ml), _i32(n_splits), _i64(T), _i32(tiles.shape[1]), _i32(tile_queries),
          _i32(heads), _i32(kv_heads), _i32(d), _i32(page_size), _i32(block_table.shape[1]), _f32(scale),
          _i32(window), _stream())


ROUTE_SMALL_TOKENS = 128


def moe_route(x: torch.Tensor, router_w: torch.Tensor, shared_gate_w: Optional[torch.Tensor], topk_w: torch.Tensor,
              topk_e: torch.Tensor, shared_gate: Optional[torch.Tensor], renormalize: bool, scale: float,
              always: int = 0) -> None:
    """Router product, softmax and top-k in float32; optional sigmoid gate of the shared expert.
    `always`: that many further slots per token after the chosen ones (topk_w and topk_e are [T, k + always]), naming
    the experts E .. E + always - 1 with the shared gate's value (or 1) as their weight: experts that every token uses."""
    T, H = x.shape
    E = router_w.shape[0]
    k = topk_w.shape[1] - always
    _need(router_w.shape == (E, H), "router weight must be [experts, hidden]")
    _need(k > 0 and always >= 0, "at least one chosen slot")
    _need(topk_w.shape == (T, k + always) and topk_w.dtype == torch.float32, "topk_w must be float32 [T, k + always]")
    _need(topk_e.shape == (T, k + always) and topk_e.dtype == torch.int32, "topk_e must be int32 [T, k + always]")
    if shared_gate_w is not None:
        _need(shared_gate_w.numel() == H, "shared gate weight must hold `hidden` numbers")
        _need(shared_gate is not None and shared_gate.dtype == torch.float32 and shared_gate.numel() >= T,
              "shared_gate must be float32 [T]")
    scratch = None
    all_bf16 = (x.dtype == torch.bfloat16 and router_w.dtype == torch.bfloat16
                and (shared_gate_w is None or shared_gate_w.dtype == torch.bfloat16))
    if T <= ROUTE_SMALL_TOKENS or all_bf16:
        # few tokens: scores go through a scratch so that many workgroups share the rows; many tokens in
        # bfloat16: the scores are a product on the matrix cores
        scratch = torch.empty((T, E + 1), dtype=torch.float32, device=x.device)
    _call("ix_moe_route", _ptr(x), _i32(_dt(x)), _ptr(router_w), _i32(_dt(router_w)), _ptr(shared_gate_w),
          _i32(_dt(shared_gate_w) if shared_gate_w is not None else F32), _ptr(topk_w), _ptr(topk_e),
          _ptr(shared_gate if shared_gate_w is not None else None), _ptr(scratch), _i64(T), _i64(H), _i32(E), _i32(k),
          _i32(1 if renormalize else 0), _f32(scale), _i32(always), _stream())


# the one-launch router: at most this many tokens, experts and bytes of one token as float32
ROUTE_ONE_LAUNCH_EXPERTS, ROUTE_ONE_LAUNCH_ROW_BYTES = 256, 40 * 1024
ROUTE_ONE_LAUNCH_TOKENS = 16
_arrival_counters: dict = {}


def _arrival_counter(device: torch.device) -> torch.Tensor:
    """Counters (one for the launch and one per token) per device that the one-launch router's workgroups count
    themselves off on; every launch leaves them zero.  Launches on one device follow one another on a stream, so
    they can share them."""
    c = _arrival_counters.get(device)
    if c is None:
        c = _arrival_counters[device] = torch.zeros(1 + ROUTE_ONE_LAUNCH_TOKENS, dtype=torch.int32, device=device)
    return c


def route_one_launch_fits(tokens: int, width: int, experts: int) -> bool:
    """Whether `moe_route_dispatch` takes these sizes.  Beyond 16 tokens `moe_route` and `moe_dispatch` are as
    fast (12.4 us both at 16 tokens of 4 experts each out of 60, 11.2 against 12.3 us at 8)."""
    return (0 < tokens <= ROUTE_ONE_LAUNCH_TOKENS and experts <= ROUTE_ONE_LAUNCH_EXPERTS
            and width * 4 <= ROUTE_ONE_LAUNCH_ROW_BYTES)


def moe_route_dispatch(x: Optional[torch.Tensor], router_w: torch.Tensor, shared_gate_w: Optional[torch.Tensor],
                       topk_w: torch.Tensor, topk_e: torch.Tensor, shared_gate: Optional[torch.Tensor],
                       renormalize: bool, scale: float, offsets: torch.Tensor, rows: torch.Tensor,
                       dest: torch.Tensor, tile_rows: int = 0, tile_map: Optional[torch.Tensor] = None,
                       norm: Optional[tuple] = None) -> None:
    """`moe_route` and `moe_dispatch` for up to 16 tokens in one launch: the router scores are spread over many
    workgroups, and the last one to finish its scores selects and groups (`route_one_launch_fits`).

    With `norm` = (h, delta, weight, eps, x_out) the norm before the feed-forward is part of the launch too
    (`x` is None then): x_out = rmsnorm(h + delta) * weight is written and routed, and h += delta."""
    if norm is not None:
        h, delta, gamma, eps, x_out = norm
        _need(x is None, "x is made by the norm")
        _need(h.dtype == torch.float32 and h.dim() == 2, "the residual stream is float32 [T, H]")
        _need(delta.shape == h.shape and x_out.shape == h.shape and delta.dtype == x_out.dtype,
              "delta and x_out must have the shape of h and one type")
        _need(gamma.numel() == h.shape[1], "the norm weight must hold `hidden` numbers")
        x = x_out
    T, H = x.shape
    E = router_w.shape[0]
    k = topk_w.shape[1]
    A = T * k
    _need(route_one_launch_fits(T, H, E), "too many tokens or experts, or too wide, for the one-launch router")
    _need(router_w.shape == (E, H), "router weight must be [experts, hidden]")
    _need(topk_w.shape == (T, k) and topk_w.dtype == torch.float32, "topk_w must be float32 [T, k]")
    _need(topk_e.shape == (T, k) and topk_e.dtype == torch.int32, "topk_e must be int32 [T, k]")
    if shared_gate_w is not None:
        _need(shared_gate_w.numel() == H, "shared gate weight must hold `hidden` numbers")
        _need(shared_gate is not None and shared_gate.dtype == torch.float32 and shared_gate.numel() >= T,
              "shared_gate must be float32 [T]")
    _is_i32(offsets, E + 1)
    _is_i32(rows, A)
    _is_i32(dest, A)
    te = tr = ti = None
    if tile_rows > 0:
        mt = moe_max_tiles(A, E, tile_rows)
        _need(tile_map is not None, "tile_map needed")
        _is_i32(tile_map, 2 * mt + 1)
        te, tr, ti = tile_map[:mt], tile_map[mt:2 * mt], tile_map[2 * mt:]
    logits = torch.empty((T, E + 1), dtype=torch.float32, device=x.device)
    router = (_ptr(router_w), _i32(_dt(router_w)), _ptr(shared_gate_w),
              _i32(_dt(shared_gate_w) if shared_gate_w is not None else F32), _ptr(logits),
              _ptr(_arrival_counter(x.device)), _i64(H), _ptr(topk_w), _ptr(topk_e),
              _ptr(shared_gate if shared_gate_w is not None else None), _ptr(offsets), _ptr(rows), _ptr(dest),
              _i32(T), _i32(E), _i32(k), _i32(1 if renormalize else 0), _f32(scale), _i32(tile_rows), _ptr(te),
              _ptr(tr), _ptr(ti), _stream())
    if norm is not None:
        _call("ix_moe_norm_route_dispatch_small", _ptr(h), _ptr(delta), _i32(_dt(x_out)), _ptr(gamma),
              _i32(_dt(gamma)), _f32(eps), _ptr(x_out), *router)
    else:
        _call("ix_moe_route_dispatch_small", _ptr(x), _i32(_dt(x)), *router)


def moe_dispatch(topk_e: torch.Tensor, offsets: torch.Tensor, rows: torch.Tensor, dest: torch.Tensor,
                 experts: int, tile_rows: int = 0, tile_map: Optional[torch.Tensor] = None) -> None:
    """Group assignments by expert: offsets [E+1], rows [A] (grouped row -> token), dest [A].
    With tile_rows > 0 also the row-tile map for the matrix-core product: `tile_map` int32
    [2 * max_tiles + 1] = tile_expert | tile_row0 | number of tiles, max_tiles = moe_max_tiles(A, E, tile_rows)."""
    T, k = topk_e.shape
    A = T * k
    _is_i32(topk_e)
    _is_i32(offsets, experts + 1)
    _is_i32(rows, A)
    _is_i32(dest, A)
    te = tr = ti = None
    if tile_rows > 0:
        mt = moe_max_tiles(A, experts, tile_rows)
        _need(tile_map is not None, "tile_map needed")
        _is_i32(tile_map, 2 * mt + 1)
        te, tr, ti = tile_map[:mt], tile_map[mt:2 * mt], tile_map[2 * mt:]
    _call("ix_moe_dispatch", _ptr(topk_e), _ptr(offsets), _ptr(rows), _ptr(dest), _i64(A), _i32(experts), _i32(k),
          _i32(tile_rows), _ptr(te), _ptr(tr), _ptr(ti), _stream())


def moe_max_tiles(assignments: int, experts: int, tile_rows: int) -> int:
    """Upper bound of the number of row tiles: every expert may end with a partial tile."""
    return max(1, min(assignments, -(-assignments // tile_rows) + experts))


def moe_grouped_mfma(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                     rows: Optional[torch.Tensor], tile_map: torch.Tensor, tile_rows: int, gate_up: bool,
                     k_split: int) -> None:
    """Grouped product on the matrix cores (bfloat16), shapes as `moe_grouped_plain`; `tile_map` from `moe_dispatch`."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if gate_up else n_out),
          "expert weight shape does not fit")
    _need(K % 8 == 0, "the reduction width must be a multiple of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, tile_rows)
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_mfma", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i32(tile_rows), _i64(n_out), _i64(K),
          _i32(1 if gate_up else 0), _i32(k_split), _stream())


def moe_grouped_dual(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                     rows: Optional[torch.Tensor], tile_map: torch.Tensor, tile_rows: int, a_s: torch.Tensor,
                     w_s: torch.Tensor, out_s: torch.Tensor, gate_up: bool) -> None:
    """`moe_grouped_mfma` (split reduction) for the routed experts and, in the same launch, the shared expert:
    out_s = a_s . w_s^T (with SwiGLU when gate_up)."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    T, n_out_s = out_s.shape
    K_s = a_s.shape[1]
    for t in (a, w, out, a_s, w_s, out_s):
        _need(t.dtype == torch.bfloat16, "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if gate_up else n_out),
          "expert weight shape does not fit")
    _need(w_s.shape == ((2 * n_out_s if gate_up else n_out_s), K_s) and a_s.shape[0] == T,
          "shared weight shape does not fit")
    _need(K % 8 == 0 and K_s % 8 == 0, "the reduction widths must be multiples of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, tile_rows)
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_dual", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i32(tile_rows), _i64(n_out), _i64(K),
          _ptr(a_s), _ptr(w_s), _ptr(out_s), _i32(T), _i64(n_out_s), _i64(K_s), _i32(1 if gate_up else 0), _stream())


_no_library_kernel = set()  # shapes that the vendor's library has no kernel for


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
    """out [T, N] = x [T, K] . w[N, K]^T, bfloat16 operands, 32-bit accumulation, out bfloat16 or float32, through the
    vendor library's C interface.  False if that library has no kernel for the shape: nothing was queued then."""
    T, K = x.shape
    N = w.shape[0]
    key = (T, N, K, out.dtype)
    if key in _no_library_kernel:
        return False
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype in (torch.bfloat16, torch.float32),
          "bfloat16 operands and a bfloat16 or float32 result")
    _need(w.dim() == 2 and w.shape[1] == K and out.shape == (T, N), "shapes do not fit")
    fn = _functions.get("ix_gemm_bf16")
    if fn is None:
        fn = _functions["ix_gemm_bf16"] = lib().ix_gemm_bf16
    rc = fn(_ptr(x), _ptr(w), _ptr(out), T, N, K, 1 if out.dtype == torch.float32 else 0, _stream())
    if rc == 2:
        _no_library_kernel.add(key)
        return False
    if rc != 0:
        raise KernelError(lib().ix_last_error().decode("utf-8", "replace"))
    return True


def linear_skinny_f32(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out float32 [T, N] = x [T, K] . w[N, K]^T for at most 64 rows, bfloat16 operands (the head of a decode step)."""
    T, K = x.shape
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.float32,
          "bfloat16 operands and a float32 result")
    _need(w.dim() == 2 and w.shape[1] == K and out.shape == (T, w.shape[0]), "shapes do not fit")
    _need(0 < T <= 64 and K % 8 == 0, "between 1 and 64 rows and a reduction width that is a multiple of 8")
    _call("ix_linear_skinny_f32", _ptr(x), _ptr(w), _ptr(out), _i32(T), _i64(w.shape[0]), _i64(K), _stream())


MOE_TILED_ROWS = 160  # rows per tile of the LDS-staged grouped product
MOE_TILED_ROWS_WIDE = 192  # ... of its wide form


def moe_tiled_rows(wide: bool) -> int:
    return MOE_TILED_ROWS_WIDE if wide else MOE_TILED_ROWS


def moe_grouped_tiled(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                      rows: Optional[torch.Tensor], tile_map: torch.Tensor, gate_up: bool, wide: bool = False) -> None:
    """Grouped product staged through LDS (bfloat16, many rows per expert); `tile_map` made for tiles of
    `moe_tiled_rows(wide)` rows.  `wide`: 256 instead of 128 weight rows per workgroup (the same sums in the same
    order; which rows share a tile, and with it where a row's sum starts, differs)."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and out.dtype == torch.bfloat16,
          "the matrix-core grouped product is bfloat16 only")
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if gate_up else n_out),
          "expert weight shape does not fit")
    _need(K % 8 == 0, "the reduction width must be a multiple of 8")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    mt = moe_max_tiles(A, E, moe_tiled_rows(wide))
    _is_i32(tile_map, 2 * mt + 1)
    _call("ix_moe_grouped_tiled", _ptr(a), _ptr(w), _ptr(out), _ptr(offsets), _ptr(rows), _ptr(tile_map[:mt]),
          _ptr(tile_map[mt:2 * mt]), _ptr(tile_map[2 * mt:]), _i32(mt), _i64(a.shape[0]), _i64(n_out), _i64(K),
          _i32(1 if gate_up else 0), _i32(1 if wide else 0), _stream())


def moe_grouped_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, offsets: torch.Tensor,
                      rows: Optional[torch.Tensor], gate_up: bool) -> None:
    """Grouped product over device offsets.  gate_up: a [T, H] gathered through `rows`,
    w [E, 2n, H], out [A, n] = silu(gate) * up.  Otherwise a [A, K], w [E, n, K], out [A, n]."""
    E = w.shape[0]
    A, n_out = out.shape
    K = a.shape[1]
    _need(w.dim() == 3 and w.shape[2] == K and w.shape[1] == (2 * n_out if gate_up else n_out),
          "expert weight shape does not fit")
    _need(out.dtype == a.dtype, "out must have the activations' dtype")
    _is_i32(offsets, E + 1)
    if rows is not None:
        _is_i32(rows, A)
    else:
        _need(a.shape[0] >= A, "a has fewer rows than out")
    _call("ix_moe_grouped_plain", _ptr(a), _i32(_dt(a)), _ptr(w), _i32(_dt(w)), _ptr(out), _ptr(offsets), _ptr(rows),
          _i64(A), _i32(E), _i64(n_out), _i64(K), _i32(1 if gate_up else 0), _stream())


def moe_combine(y: torch.Tensor, dest: torch.Tensor, topk_w: torch.Tensor, shared: Optional[torch.Tensor],
                shared_gate: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[t] = sum_s topk_w[t, s] * y[dest[t, s]] (+ shared_gate[t] * shared[t])."""
    T, k = topk_w.shape
    H = y.shape[1]
    _need(out.shape == (T, H) and out.dtype == y.dtype, "out mismatch")
    _need(y.shape[0] >= T * k, "y has too few rows")
    _is_i32(dest, T * k)
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == y.dtype, "shared mismatch")
    _call("ix_moe_combine", _ptr(y), _i32(_dt(y)), _ptr(dest), _ptr(topk_w), _ptr(shared),
          _ptr(shared_gate if shared is not None else None), _ptr(out), _i64(T), _i64(H), _i32(k), _stream())


def moe_combine_add_rmsnorm(h: torch.Tensor, y: torch.Tensor, dest: torch.Tensor, topk_w: torch.Tensor,
                            shared: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor], weight: torch.Tensor,
                            out: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """`moe_combine` followed by `add_rmsnorm` in one pass: h += sum; out = rmsnorm(h) * weight."""
    T, k = topk_w.shape
    H = h.shape[1]
    _need(h.dtype == torch.float32 and h.shape[0] == T, "the residual stream is float32 [T, H]")
    _need(y.shape[1] == H and y.shape[0] >= T * k and out.dtype == y.dtype and out.shape[1] == H, "shape mismatch")
    _need(weight.numel() == H, "norm weight length differs")
    _is_i32(dest, T * k)
    n_out = out.shape[0]
    if rows is None:
        _need(n_out == T, "out must have a row per token")
    else:
        _is_i32(rows, n_out)
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == y.dtype, "shared mismatch")
    _call("ix_moe_combine_add_rmsnorm", _ptr(h), _ptr(y), _i32(_dt(y)), _ptr(dest), _ptr(topk_w), _ptr(shared),
          _ptr(shared_gate if shared is not None else None), _ptr(weight), _i32(_dt(weight)), _ptr(out), _ptr(rows),
          _i64(n_out), _i64(H), _i32(k), _f32(eps), _stream())


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(out, R)
    if V > 4 * 4096 and R < 256:  # few long rows: two stages, so that they still fill the machine
        chunks = -(-V // 4096)
        part_v = torch.empty((R, chunks), dtype=torch.float32, device=logits.device)
        part_i = torch.empty((R, chunks), dtype=torch.int32, device=logits.device)
        _call("ix_argmax_two_stage", _ptr(logits), _ptr(out), _ptr(part_v), _ptr(part_i), _i64(R), _i64(V), _stream())
        return
    _call("ix_argmax", _ptr(logits), _ptr(out), _i64(R), _i64(V), _stream())


def sample(logits: torch.Tensor, out: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           top_k: torch.Tensor, min_p: torch.Tensor, rng_key: torch.Tensor, rng_counter: torch.Tensor,
           advance: bool = False) -> None:
    """Row r's draw is number rng_counter[r] of the stream rng_key[r]; with `advance` the kernel leaves
    rng_counter[r] + 1 there."""
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(out, R)
    _is_i32(top_k, R)
    for t in (temperature, top_p, min_p):
        _need(t.dtype == torch.float32 and t.numel() >= R, "sampling parameters must be float32 [rows]")
    for t in (rng_key, rng_counter):
        _need(t.dtype == torch.int64 and t.numel() >= R, "rng key and counter must be int64 [rows]")
    _call("ix_sample", _ptr(logits), _ptr(out), _ptr(temperature), _ptr(top_p), _ptr(top_k), _ptr(min_p),
          _ptr(rng_key), _ptr(rng_counter), _i32(1 if advance else 0), _i64(R), _i64(V), _stream())


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, chosen_lp: torch.Tensor, top_ids: torch.Tensor,
             top_lp: torch.Tensor) -> None:
    """Log-probability of each row's chosen token and of its n_top most probable tokens (n_top = top_ids.shape[1])."""
    R, V = logits.shape
    n_top = top_ids.shape[1]
    _need(logits.dtype == torch.float32, "logits must be float32")
    _is_i32(chosen, R)
    _need(chosen_lp.dtype == torch.float32 and chosen_lp.numel() >= R, "chosen_lp must be float32 [rows]")
    _need(top_ids.shape == (R, n_top) and top_ids.dtype == torch.int32, "top_ids must be int32 [rows, n_top]")
    _need(top_lp.shape == (R, n_top) and top_lp.dtype == torch.float32, "top_lp must be float32 [rows, n_top]")
    _call("ix_logprobs", _ptr(logits), _ptr(chosen), _ptr(chosen_lp), _ptr(top_ids), _ptr(top_lp), _i64(R), _i64(V),
          _i32(n_top), _stream())


def apply_penalties(logits: torch.Tensor, hist_begin: torch.Tensor, hist_ids: torch.Tensor,
                    hist_counts: torch.Tensor, presence: torch.Tensor, frequency: torch.Tensor,
                    repetition: torch.Tensor, mask_begin: torch.Tensor, mask_ids: torch.Tensor) -> None:
    """In place on float32 logits [R, V]; histories and masks in CSR form (begin arrays hold R + 1 entries)."""
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits must be float32")
    for t in (hist_begin, mask_begin):
        _is_i32(t, R + 1)
    for t in (hist_ids, hist_counts, mask_ids):
        _is_i32(t)
    for t in (presence, frequency, repetition):
        _need(t.dtype == torch.float32 and t.numel() >= R, "penalties must be float32 [rows]")
    _call("ix_apply_penalties", _ptr(logits), _ptr(hist_begin), _ptr(hist_ids), _ptr(hist_counts), _ptr(presence),
          _ptr(frequency), _ptr(repetition), _ptr(mask_begin), _ptr(mask_ids), _i64(R), _i64(V), _stream())


def measured_ceilings(device=None, read_bytes: int = 4 << 30) -> dict:
    """What this machine gives a kernel that only reads memory (GB/s, over a buffer far larger than any cache)
    and one that only issues bfloat16 matrix-core products (TFLOP/s): the measured ceilings that results are
    priced against beside the published peaks.  Takes a few tens of milliseconds and `read_bytes` of memory."""
    device = torch.device(device or "cuda:0")
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    buf = torch.empty(read_bytes // 4, dtype=torch.int32, device=device)
    buf.fill_(1)
    out = torch.zeros(1024, dtype=torch.int32, device=device)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = 0.0
    for blocks in (cus * 8, cus * 16, cus * 32):
        _call("ix_probe_read", _ptr(buf), _i64(read_bytes), _ptr(out), _i32(blocks), _i32(1), _stream())  # warm
        start.record()
        _call("ix_probe_read", _ptr(buf), _i64(read_bytes), _ptr(out), _i32(blocks), _i32(4), _stream())
        stop.record()
        stop.synchronize()
        best_read = max(best_read, 4 * read_bytes / (start.elapsed_time(stop) * 1e-3) / 1e9)
    del buf
    sink = torch.zeros(1, dtype=torch.float32, device=device)
    flops = ctypes.c_double(0.0)
    best_mfma = 0.0
    for waves_per_simd in (2, 4):
        blocks, iters = cus * waves_per_simd, 100000
        _call("ix_probe_mfma", _i32(blocks), _i32(200), _ptr(sink), ctypes.byref(flops), _stream())  # warm
        start.record()
        _call("ix_probe_mfma", _i32(blocks), _i32(iters), _ptr(sink), ctypes.byref(flops), _stream())
        stop.record()
        stop.synchronize()
        best_mfma = max(best_mfma, flops.value / (start.elapsed_time(stop) * 1e-3) / 1e12)
    return {"hbm_read_gbs": round(best_read, 1), "mfma_bf16_tflops": round(best_mfma, 1)}
