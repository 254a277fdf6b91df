"""Each part of a layer alone (norm, attention with its position encoding, dense and
expert feed-forward, the block) against the plain implementation's function for it."""
import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PARAMS = [("float32", 2e-5), ("bfloat16", 2e-2)]


def make_ctx(rt, q_lens, seq_lens, page_size, pages, groups=1):
    """A step context for requests with the given new and total lengths (pages handed out in order)."""
    from inferx_amd.cache.manager import CacheManager, GroupLayout
    from inferx_amd.engine.batch import build_step_batch
    from inferx_amd.engine.runner import _pack
    from inferx_amd.engine.runtime import StepContext
    cache = CacheManager([GroupLayout(0)] * groups, [pages] * groups, page_size, len(q_lens), pages * page_size)
    entries = []
    for i, (n, L) in enumerate(zip(q_lens, seq_lens)):
        cache.add(i)
        if L > n:
            cache.reserve(i, L - n)
            cache.commit(i, L - n)
        entries.append((i, [0] * n, list(range(n))))
    batch = build_step_batch(cache, entries)
    sizes, flat = _pack(batch)
    dev = torch.from_numpy(flat).to(DEV)
    views, at = [], 0
    for n in sizes:
        views.append(dev[at:at + n])
        at += n
    S, G = len(q_lens), groups
    return StepContext(rt=rt, num_tokens=batch.num_tokens, num_requests=S, token_ids=views[0], positions=views[1],
                       seq_of_token=views[2], q_start=views[3], seq_lens=views[4], state_slots=views[5],
                       logits_rows=views[6], slots=views[7:7 + G],
                       block_tables=[views[7 + G + g].view(S, -1) for g in range(G)], host=batch,
                       one_token_each=batch.one_token_each), batch


def tensors_for(part, rt, seed=0, std=None):
    out = {}
    for i, p in enumerate(part.param_specs()):
        g = torch.Generator().manual_seed(seed * 1000 + i)
        t = torch.ones(p.shape) if p.init == "ones" else torch.randn(p.shape, generator=g) * (std or p.std)
        out[p.name] = t.to(rt.dtype)
    return out


def err(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max()) / float(want.abs().max())


@pytest.mark.parametrize("dtype,tol", PARAMS)
def test_rmsnorm_part(dtype, tol):
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_part
    from inferx_amd.config import PartSpec
    rt = Runtime(dtype)
    part = build_part("norm", PartSpec("rmsnorm", {"width": 72, "eps": 1e-5}))
    w = {"weight": (torch.randn(72, generator=torch.Generator().manual_seed(1)) * 0.5 + 1).to(rt.dtype)}
    part.bind({k: v.to(DEV) for k, v in w.items()}, rt)
    ctx, _ = make_ctx(rt, [5], [5], 16, 4)
    h = torch.randn(5, 72, generator=torch.Generator().manual_seed(2)).to(DEV)
    delta = torch.randn(5, 72, generator=torch.Generator().manual_seed(3)).to(rt.dtype).to(DEV)
    want_h = h.double().cpu() + delta.double().cpu()
    out = part.forward(ctx, h, delta)
    assert err(out, pm.rms_norm(want_h, w["weight"].double(), 1e-5)) < tol
    assert err(h, want_h) < 1e-6


@pytest.mark.parametrize("dtype,tol", PARAMS)
@pytest.mark.parametrize("heads,kv,d,window,bias,rotated", [
    (4, 2, 16, 0, True, None), (3, 1, 32, 7, True, None), (6, 3, 48, 0, False, None),
    # a part of every head rotated: the trailing half, a stretch in the middle, the leading quarter of large heads
    (4, 2, 16, 0, True, (8, 8)), (3, 1, 32, 7, False, (6, 20)), (2, 2, 128, 0, True, (0, 32))])
@pytest.mark.parametrize("out_bias", [False, True])
def test_attention_part_whole_and_in_two_steps(dtype, tol, heads, kv, d, window, bias, rotated, out_bias):
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import CacheBinding, Runtime
    from inferx_amd.parts import build_part
    rt = Runtime(dtype)
    H, theta, T = 40, 10000.0, 37
    begin, dim = rotated or (0, d)
    spec = PartSpec("attention", {"hidden_size": H, "num_heads": heads, "num_kv_heads": kv, "head_dim": d,
                                  "qkv_bias": bias, "window": window, "out_bias": out_bias,
                                  "position": PartSpec("rope", {"theta": theta, "rotary_dim": dim, "begin": begin}),
                                  "init_std": 0.2})
    part = build_part("mixer", spec)
    w = tensors_for(part, rt, seed=4)
    part.bind({k: v.to(DEV) for k, v in w.items()}, rt)
    x = (torch.randn(T, H, generator=torch.Generator().manual_seed(5))).to(rt.dtype)
    # plain: projections, bias, rotation, attention, output projection (tests/plain_model.py forward())
    wd = {k: v.double() for k, v in w.items()}
    xd = x.double()
    q, k, v = xd @ wd["q_proj.weight"].T, xd @ wd["k_proj.weight"].T, xd @ wd["v_proj.weight"].T
    if bias:
        q, k, v = q + wd["q_proj.bias"], k + wd["k_proj.bias"], v + wd["v_proj.bias"]
    pos = torch.arange(T)
    att = pm.attention(pm.apply_rope_part(q.view(T, heads, d), pos, theta, begin, dim),
                       pm.apply_rope_part(k.view(T, kv, d), pos, theta, begin, dim), v.view(T, kv, d), pos, d ** -0.5,
                       window)
    want = att.reshape(T, heads * d) @ wd["o_proj.weight"].T
    if out_bias:
        want = want + wd["o_proj.bias"]

    def run(splits):
        pages, page = 4, 16
        cache = CacheBinding(group=0, arrays=dict(k=torch.zeros(pages, kv, page, d, dtype=rt.dtype, device=DEV),
                                                v=torch.zeros(pages, kv, d, page, dtype=rt.dtype, device=DEV)))
        outs, done = [], 0
        for n in splits:
            ctx, _ = make_ctx(rt, [n], [done + n], page, pages)
            outs.append(part.forward(ctx, x[done:done + n].to(DEV), cache))
            done += n
        return torch.cat(outs)

    assert err(run([T]), want) < tol
    assert err(run([20, 2, 14, 1]), want) < tol


@pytest.mark.parametrize("heads,kv,d,window,q_lens,seq_lens,expect", [
    (16, 16, 128, 0, [128], [7000], "slices"),                  # few tiles on a long context: keys in slices
    (28, 4, 128, 0, [1, 300, 1, 2], [5000, 6500, 900, 40], "slices, grouped beside"),  # ... beside requests of one
                                                                # and two tokens, served per key/value head
    (16, 16, 48, 0, [130, 1], [400, 77], "one kernel"),         # few tiles of 64, short context
    (16, 16, 64, 0, [130, 1], [400, 77], "portion and tokens"), # (a head of two 32s: a tile of 128 and a token beside)
    (16, 16, 112, 0, [2100], [2100], "pairs"),                  # many tiles of 64, in pairs
    (16, 16, 64, 0, [2100], [2100], "tiles"),                   # tiles of 128, a workgroup each
    (8, 2, 64, 512, [200, 1, 1], [3000, 2000, 10], "portion and tokens"),  # a window; the one-token requests grouped
    (8, 2, 80, 512, [200, 1, 1], [3000, 2000, 10], "two launches"),  # (no tiles of 128 for this head size)
    (28, 4, 128, 0, [64, 1, 1, 1], [500, 3000, 200, 10], "two launches"),  # a small step: no LDS-sharing kernel
    (28, 4, 128, 0, [1, 1, 1], [3000, 17, 600], "grouped"),     # one token each
])
def test_attention_kernels_chosen_by_the_step(heads, kv, d, window, q_lens, seq_lens, expect):
    """`PagedAttention.attend` on steps of realistic head counts and contexts: whichever kernels the step's plan
    chooses (portions in tiles, in pairs or with their keys in slices; few-token requests beside them), the result
    is float64 attention per request."""
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import CacheBinding, Runtime
    from inferx_amd.parts import build_part
    rt = Runtime("bfloat16")
    part = build_part("mixer", PartSpec("attention", {"hidden_size": 64, "num_heads": heads, "num_kv_heads": kv,
                                                      "head_dim": d, "window": window}))
    page = 16
    pages = sum(-(-L // page) for L in seq_lens) + 2
    ctx, batch = make_ctx(rt, q_lens, seq_lens, page, pages)
    table = batch.block_tables[0].reshape(len(q_lens), -1)
    k_cache = torch.zeros(pages, kv, page, d, dtype=torch.bfloat16)
    v_cache = torch.zeros(pages, kv, d, page, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(12)
    qs, wants = [], []
    for s, (n, L) in enumerate(zip(q_lens, seq_lens)):
        k = torch.randn(L, kv, d, generator=g).bfloat16()
        v = torch.randn(L, kv, d, generator=g).bfloat16()
        q = torch.randn(n, heads, d, generator=g).bfloat16()
        for j in range(-(-L // page)):
            rows = slice(j * page, min(L, (j + 1) * page))
            m = rows.stop - rows.start
            k_cache[int(table[s, j]), :, :m, :] = k[rows].transpose(0, 1)
            v_cache[int(table[s, j]), :, :, :m] = v[rows].permute(1, 2, 0)
        qs.append(q)
        wants.append(None)
        # float64 attention of this request's new rows over all its keys
        kk, vv = k.double().repeat_interleave(heads // kv, 1), v.double().repeat_interleave(heads // kv, 1)
        sc = torch.einsum("qhd,khd->hqk", q.double(), kk) * d ** -0.5
        qpos, kpos = torch.arange(L - n, L)[:, None], torch.arange(L)[None, :]
        ok = kpos <= qpos
        if window > 0:
            ok &= kpos >= qpos + 1 - window
        wants[-1] = torch.einsum("hqk,khd->qhd", torch.softmax(sc.masked_fill(~ok[None], -float("inf")), -1), vv)
    q = torch.cat(qs).to(DEV)
    out = torch.full_like(q, float("nan"))
    part.attend(ctx, q, CacheBinding(group=0, arrays=dict(k=k_cache.to(DEV), v=v_cache.to(DEV))), out)
    assert err(out, torch.cat(wants)) < 1.5e-2
    # the plan that attend() followed (memoised in the step's context)
    from inferx_amd.parts import attention
    if expect == "grouped":
        assert attention.query_tiles(ctx, window, heads, d, kv)[3]
    else:
        tile = attention.WIDE_PREFILL_TILE if d % 32 == 0 else attention.PREFILL_TILE
        lds, waves = attention.mixed_step_plan(ctx, window, heads, kv, True, tile)
        if expect == "one kernel":
            assert lds is None and len(waves) == 1 and waves[0][0] is None and not waves[0][4]
        elif expect == "two launches":
            assert lds is None and [w[4] for w in waves] == [True, False] and all(w[0] is not None for w in waves)
        elif expect == "pairs":
            assert lds[2] == 1 and not waves and int(lds[1][1].max()) >= 0
        elif expect == "tiles":
            assert lds[2] == 1 and not waves and int(lds[1][1].max()) < 0 and int(lds[0][2].max()) == 128
        elif expect == "portion and tokens":
            assert lds is not None and lds[2] == 1 and len(waves) == 1 and waves[0][4] == (heads > kv)
        elif expect == "slices":
            assert lds[2] > 1 and not waves
        else:
            assert lds[2] > 1 and len(waves) == 1 and waves[0][4]


@pytest.mark.parametrize("dtype,tol", PARAMS)
def test_dense_mlp_part(dtype, tol):
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_part
    rt = Runtime(dtype)
    part = build_part("feed_forward", PartSpec("dense_mlp", {"hidden_size": 72, "width": 104, "init_std": 0.2}))
    w = tensors_for(part, rt, seed=6)
    part.bind({k: v.to(DEV) for k, v in w.items()}, rt)
    ctx, _ = make_ctx(rt, [9], [9], 16, 4)
    x = torch.randn(9, 72, generator=torch.Generator().manual_seed(7)).to(rt.dtype)
    want = pm.gated_mlp(x.double(), w["gate_proj.weight"].double(), w["up_proj.weight"].double(),
                        w["down_proj.weight"].double())
    assert err(part.forward(ctx, x.to(DEV)), want) < tol


@pytest.mark.parametrize("dtype,tol", PARAMS)
@pytest.mark.parametrize("H,E,k,mi,si,renorm,gated", [(64, 4, 2, 32, 64, False, True), (96, 8, 3, 48, 80, True, True),
                                                      (72, 5, 1, 40, 0, False, True), (64, 6, 6, 32, 48, True, False),
                                                      (64, 1, 1, 32, 0, False, True), (64, 6, 3, 32, 96, True, False)])
# 7, 29: the few-token path (experts and shared expert in one launch); 40, 300: steps of middling size, where a shared
# expert whose width is a multiple of the experts' (the first case, gated; the last, not) rides along as pieces that
# every token chooses, through the streaming kernel (40) and the LDS-staged one (300)
@pytest.mark.parametrize("T", [300, 40, 29, 7])
def test_moe_part(dtype, tol, H, E, k, mi, si, renorm, gated, T):
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_part
    rt = Runtime(dtype)
    part = build_part("feed_forward", PartSpec("moe", {
        "hidden_size": H, "num_experts": E, "top_k": k, "expert_width": mi, "shared_width": si,
        "shared_gated": gated, "renormalize": renorm, "init_std": 0.15}))
    w = tensors_for(part, rt, seed=8)
    part.bind({n: v.to(DEV) for n, v in w.items()}, rt)
    assert part.shared_pieces == (si // mi if (si and si % mi == 0 and dtype == "bfloat16") else 0)
    ctx, _ = make_ctx(rt, [T], [T], 16, T // 16 + 2)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(9)).to(rt.dtype)
    wd = {"m." + n: v.double() for n, v in w.items()}
    if si and not gated:  # an ungated shared expert adds exactly its output: sigmoid(+inf) = 1
        wd["m.shared_expert_gate.weight"] = torch.full((1, H), 1e4, dtype=torch.float64) * torch.sign(x.double().sum(0))
        want = pm.moe_block(x.double(), {n: v for n, v in wd.items() if "shared" not in n}, "m.", E, k, renorm, 0) + \
            pm.gated_mlp(x.double(), wd["m.shared_expert.gate_proj.weight"], wd["m.shared_expert.up_proj.weight"],
                         wd["m.shared_expert.down_proj.weight"])
    else:
        want = pm.moe_block(x.double(), wd, "m.", E, k, renorm, si)
    from inferx_amd.parts import resolve_delta
    lazy = part.forward(ctx, x.to(DEV))
    got = resolve_delta(ctx, lazy)
    assert err(got, want) < tol
    # the routing itself, exactly (float32 scores): experts and weights per slot
    topk_w, topk_e, _ = part.route(ctx, x.to(DEV))
    want_w, want_e = pm.route(x.double(), wd["m.gate.weight"], k, renorm)
    assert torch.equal(topk_e.cpu().long(), want_e)
    assert err(topk_w, want_w) < 1e-5
    # repeat runs are bitwise equal (reference: tests/kernel/moe_test.cc:972-1046)
    again = resolve_delta(ctx, part.forward(ctx, x.to(DEV)))
    assert torch.equal(got.view(torch.int16 if dtype == "bfloat16" else torch.int32),
                       again.view(torch.int16 if dtype == "bfloat16" else torch.int32))


def test_moe_part_with_wide_expert_tiles():
    """The expert products' wide form (chosen by the part from a width of 3,072 on; forced here at a small one)
    gives the bits of the narrow form, with the shared expert on the main stream."""
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_part, resolve_delta
    from inferx_amd.parts import moe as moe_part
    rt = Runtime("bfloat16")
    H, E, k, mi, si, T = 64, 4, 2, 32, 64, 300
    assert build_part("feed_forward", PartSpec("moe", {"hidden_size": moe_part.WIDE_TILES_WIDTH, "num_experts": 2,
                                                       "top_k": 1, "expert_width": 8})).wide_tiles
    part = build_part("feed_forward", PartSpec("moe", {
        "hidden_size": H, "num_experts": E, "top_k": k, "expert_width": mi, "shared_width": si, "init_std": 0.15}))
    assert not part.wide_tiles
    w = tensors_for(part, rt, seed=8)
    part.bind({n: v.to(DEV) for n, v in w.items()}, rt)
    ctx, _ = make_ctx(rt, [T], [T], 16, 32)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(9)).to(rt.dtype)
    narrow = resolve_delta(ctx, part.forward(ctx, x.to(DEV)))
    part.wide_tiles = True
    wide = resolve_delta(ctx, part.forward(ctx, x.to(DEV)))
    assert torch.equal(narrow.view(torch.int16), wide.view(torch.int16))
    wd = {"m." + n: v.double() for n, v in w.items()}
    assert err(wide, pm.moe_block(x.double(), wd, "m.", E, k, False, si)) < 2e-2


def test_shared_expert_beside_the_routed_ones():
    """A prompt portion: the shared expert runs on a second stream beside the routed experts.  The sum is bit for
    bit that of one stream, also when the calls follow one another without a wait (memory of one call is given
    out again to the next) and under work that keeps the main stream busy."""
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_part, moe, resolve_delta
    rt = Runtime("bfloat16")
    H, T = 136, 640
    part = build_part("feed_forward", PartSpec("moe", {
        "hidden_size": H, "num_experts": 8, "top_k": 2, "expert_width": 72, "shared_width": 200,
        "shared_gated": True, "renormalize": False, "init_std": 0.15}))
    part.bind({n: v.to(DEV) for n, v in tensors_for(part, rt, seed=3).items()}, rt)
    ctx, _ = make_ctx(rt, [T], [T], 16, 41)
    xs = [torch.randn(T, H, generator=torch.Generator().manual_seed(s)).to(rt.dtype).to(DEV) for s in range(6)]
    assert part._tile_rows(ctx, xs[0]) == ops_tiled_rows() and rt.can_run_beside()
    threshold = moe.SHARED_BESIDE_TOKENS
    try:
        moe.SHARED_BESIDE_TOKENS = 1 << 30
        want = [resolve_delta(ctx, part.forward(ctx, x)) for x in xs]
        moe.SHARED_BESIDE_TOKENS = 256
        assert rt._side_stream is None
        busy = torch.randn(2048, 2048, device=DEV)
        got = []
        for x in xs:  # no wait between the calls
            busy = busy @ busy * 1e-3
            got.append(resolve_delta(ctx, part.forward(ctx, x)))
        assert rt._side_stream is not None
    finally:
        moe.SHARED_BESIDE_TOKENS = threshold
    torch.cuda.synchronize()
    for g, w in zip(got, want):
        assert torch.equal(g.view(torch.int16), w.view(torch.int16))


def ops_tiled_rows():
    from inferx_amd import ops
    return ops.MOE_TILED_ROWS


@pytest.mark.parametrize("dtype,tol", PARAMS)
def test_norm_fuses_the_expert_sum(dtype, tol):
    """The norm forms a lazy expert sum itself: same stream and same output as sum, add, norm one after the other."""
    from inferx_amd.config import PartSpec
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import LazyDelta, build_part, resolve_delta
    rt = Runtime(dtype)
    H, T = 96, 21
    moe = build_part("feed_forward", PartSpec("moe", {"hidden_size": H, "num_experts": 8, "top_k": 3,
                                                      "expert_width": 48, "shared_width": 80, "init_std": 0.15}))
    moe.bind({n: v.to(DEV) for n, v in tensors_for(moe, rt, seed=11).items()}, rt)
    norm = build_part("norm", PartSpec("rmsnorm", {"width": H, "eps": 1e-5}))
    norm.bind({"weight": (torch.rand(H) + 0.5).to(rt.dtype).to(DEV)}, rt)
    ctx, _ = make_ctx(rt, [T], [T], 16, 4)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(12)).to(rt.dtype).to(DEV)
    h0 = torch.randn(T, H, generator=torch.Generator().manual_seed(13)).to(DEV)
    lazy = moe.forward(ctx, x)
    assert isinstance(lazy, LazyDelta)
    h1, h2 = h0.clone(), h0.clone()
    fused = norm.forward(ctx, h1, lazy)
    plain = norm.forward(ctx, h2, resolve_delta(ctx, lazy))
    assert err(h1, h2) < (1e-6 if dtype == "float32" else 1e-2)
    assert err(fused, plain) < (1e-5 if dtype == "float32" else 1e-2)
    rows = torch.tensor([T - 1, 0, 5, 5], dtype=torch.int32, device=DEV)
    h3 = h0.clone()
    picked = norm.forward(ctx, h3, lazy, rows=rows)
    assert torch.equal(h3, h0) and err(picked, plain[rows.long()]) < (1e-5 if dtype == "float32" else 1e-2)


def test_registry_errors():
    from inferx_amd.config import PartSpec
    from inferx_amd.parts import build_part
    with pytest.raises(KeyError, match="no mixer registered as 'nonesuch'"):
        build_part("mixer", PartSpec("nonesuch"))
    part = build_part("mixer", PartSpec("attention", {"hidden_size": 32, "num_heads": 2, "num_kv_heads": 2, "head_dim": 16,
                                                      "position": PartSpec("rope", {"theta": 1e4, "rotary_dim": 8})}))
    assert part.rotated == (0, 8)
    with pytest.raises(ValueError, match="rotates elements 12 to 20 of heads of 16"):
        build_part("mixer", PartSpec("attention", {"hidden_size": 32, "num_heads": 2, "num_kv_heads": 2, "head_dim": 16,
                                                   "position": PartSpec("rope", {"theta": 1e4, "rotary_dim": 8, "begin": 12})}))
