"""Embedding, norm, SwiGLU product, rotary table, bias + rotation + cache append, greedy and
temperature sampling, penalties: each kernel alone against a PyTorch reference."""
import math

import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def rel_err(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max()) / max(float(want.abs().max()), 1e-30)


def tol(dtype):
    return 2e-6 if dtype == torch.float32 else 8e-3


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    from inferx_amd import ops
    table = rnd(301, 72, dtype=dtype)
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32, device=DEV)
    h = torch.empty(5, 72, device=DEV)
    ops.embed(h, table, ids)
    assert torch.equal(h.cpu(), table.float().cpu()[ids.long().cpu()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("T,H,eps", [(5, 72, 1e-5), (3, 2048, 1e-6), (2, 5000, 1e-6)])
def test_add_rmsnorm(dtype, wdtype, T, H, eps):
    from inferx_amd import ops
    h0, delta, w = rnd(T, H), rnd(T, H, seed=1, dtype=dtype), rnd(H, seed=2, dtype=wdtype)
    h = h0.clone()
    out = torch.empty(T, H, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h, delta, w, out, eps)
    v = h0.double().cpu() + delta.double().cpu()
    assert rel_err(h, v) < 1e-6  # the residual stream carries the sum, in float32
    assert rel_err(out, pm.rms_norm(v, w.double().cpu(), eps)) < tol(dtype)
    # no delta; and picked rows (a row may be asked for twice; h is then left alone)
    h = h0.clone()
    ops.add_rmsnorm(h, None, w, out, eps)
    assert torch.equal(h, h0) and rel_err(out, pm.rms_norm(h0.double().cpu(), w.double().cpu(), eps)) < tol(dtype)
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, H, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h, delta, w, picked, eps, rows)
    assert torch.equal(h, h0)
    assert rel_err(picked, pm.rms_norm(v, w.double().cpu(), eps)[rows.long().cpu()]) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    from inferx_amd import ops
    gu = rnd(7, 2 * 104, dtype=dtype, scale=3.0)
    out = torch.empty(7, 104, dtype=dtype, device=DEV)
    ops.silu_mul(gu, out)
    g, u = gu.double().cpu()[:, :104], gu.double().cpu()[:, 104:]
    assert rel_err(out, pm.silu(g) * u) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,width", [(33, 1408), (5, 24), (64, 100)])
def test_silu_mul_sizes(dtype, T, width):
    """Widths that take the 16-byte path (multiples of 8) and one that does not."""
    from inferx_amd import ops
    gu = rnd(T, 2 * width, dtype=dtype, scale=3.0)
    out = torch.empty(T, width, dtype=dtype, device=DEV)
    ops.silu_mul(gu, out)
    g, u = gu.double().cpu()[:, :width], gu.double().cpu()[:, width:]
    assert rel_err(out, pm.silu(g) * u) < tol(dtype)


@pytest.mark.parametrize("theta,d", [(10000.0, 16), (1e6, 128), (50000.0, 48)])
def test_rope_table(theta, d):
    from inferx_amd import ops
    from inferx_amd.parts.rope import Rotary
    pos = torch.tensor([0, 1, 2, 17, 255, 4095, 32767], dtype=torch.int32, device=DEV)
    inv = Rotary(theta, d).frequencies().to(DEV)
    assert torch.equal(inv.cpu().double(), pm.rope_frequencies(theta, d))
    table = torch.empty(len(pos), d // 2, 2, device=DEV)
    ops.rope_table(table, pos, inv)
    angle = (pos.cpu().float()[:, None] * inv.cpu()[None, :]).double()
    assert float((table[..., 0].cpu().double() - torch.cos(angle)).abs().max()) < 2e-6
    assert float((table[..., 1].cpu().double() - torch.sin(angle)).abs().max()) < 2e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,d,page,bias,rotated", [
    (4, 2, 16, 16, True, None), (3, 1, 32, 16, True, None), (6, 3, 48, 32, False, None), (16, 16, 128, 16, True, None),
    # only a part of every head is rotated, the rest passes through
    (4, 2, 16, 16, True, (8, 8)), (3, 1, 32, 16, False, (6, 20)), (5, 5, 128, 16, True, (0, 64)), (2, 1, 48, 32, True, (46, 2)),
    (3, 3, 32, 16, True, (7, 12)), (2, 2, 18, 16, False, (1, 16))])
def test_qkv_rope_append(dtype, heads, kv, d, page, bias, rotated):
    from inferx_amd import ops
    from inferx_amd.parts.rope import Rotary
    T, pages, theta = 9, 5, 10000.0
    width = (heads + 2 * kv) * d
    qkv = rnd(T, width, dtype=dtype)
    b = rnd(width, seed=1, dtype=dtype) if bias else None
    pos = torch.tensor([3, 4, 5, 6, 0, 1, 40, 41, 42], dtype=torch.int32, device=DEV)
    slots = torch.tensor([page * 2 + 3, page * 2 + 4, page * 2 + 5, page * 2 + 6, 0, 1, page * 4 + 8, page * 4 + 9,
                          page * 1 + 0], dtype=torch.int32, device=DEV)
    begin, dim = rotated or (0, d)
    table = torch.empty(T, dim // 2, 2, device=DEV)
    ops.rope_table(table, pos, Rotary(theta, dim).frequencies().to(DEV))
    q = torch.empty(T, heads, d, dtype=dtype, device=DEV)
    kc = torch.zeros(pages, kv, page, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, kv, d, page, dtype=dtype, device=DEV)
    ops.qkv_rope_append(qkv, b, table, slots, q, kc, vc, heads, kv, d, rotated=rotated)
    x = qkv.double().cpu() + (b.double().cpu() if bias else 0)
    wq = pm.apply_rope_part(x[:, :heads * d].view(T, heads, d), pos.cpu(), theta, begin, dim)
    wk = pm.apply_rope_part(x[:, heads * d:(heads + kv) * d].view(T, kv, d), pos.cpu(), theta, begin, dim)
    wv = x[:, (heads + kv) * d:].view(T, kv, d)
    assert rel_err(q, wq) < tol(dtype)
    for t in range(T):
        pg, off = int(slots[t]) // page, int(slots[t]) % page
        assert rel_err(kc[pg, :, off, :], wk[t]) < tol(dtype)
        assert rel_err(vc[pg, :, :, off], wv[t]) < tol(dtype)
    written = torch.zeros(pages, page, dtype=torch.bool)
    for t in range(T):
        written[int(slots[t]) // page, int(slots[t]) % page] = True
    assert float(kc.float().abs().sum(dim=(1, 3)).cpu()[~written].sum()) == 0  # nothing else was touched
    # no rotation table: q and k pass through; no caches: only q is written
    q2 = torch.empty_like(q)
    ops.qkv_rope_append(qkv, b, None, None, q2, None, None, heads, kv, d)
    assert rel_err(q2, x[:, :heads * d].view(T, heads, d)) < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,d,page,bias", [(4, 2, 16, 16, True), (5, 5, 128, 16, True), (6, 3, 48, 32, False)])
def test_qkv_rope_append_many_tokens(dtype, heads, kv, d, page, bias):
    """Portions of two requests, each starting in the middle of a page and running over several pages that
    do not follow each other in the pool (the values of many tokens are written by a kernel of their own)."""
    from inferx_amd import ops
    from inferx_amd.parts.rope import Rotary
    theta, pages = 10000.0, 24
    starts, counts = [5, page + 3], [4 * page + 7, 3 * page - 2]
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(5)).tolist()
    tables = [order[:8], order[8:16]]
    pos = torch.tensor([p0 + i for p0, n in zip(starts, counts) for i in range(n)], dtype=torch.int32)
    slot_list = [tables[r][(p0 + i) // page] * page + (p0 + i) % page
                 for r, (p0, n) in enumerate(zip(starts, counts)) for i in range(n)]
    slot_list[3] = -1  # one token that writes nothing
    T, width = len(slot_list), (heads + 2 * kv) * d
    slots = torch.tensor(slot_list, dtype=torch.int32, device=DEV)
    qkv = rnd(T, width, dtype=dtype)
    b = rnd(width, seed=1, dtype=dtype) if bias else None
    table = torch.empty(T, d // 2, 2, device=DEV)
    ops.rope_table(table, pos.to(DEV), Rotary(theta, d).frequencies().to(DEV))
    q = torch.empty(T, heads, d, dtype=dtype, device=DEV)
    kc = torch.zeros(pages, kv, page, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, kv, d, page, dtype=dtype, device=DEV)
    ops.qkv_rope_append(qkv, b, table, slots, q, kc, vc, heads, kv, d)
    x = qkv.double().cpu() + (b.double().cpu() if bias else 0)
    wq = pm.apply_rope(x[:, :heads * d].view(T, heads, d), pos, theta)
    wk = pm.apply_rope(x[:, heads * d:(heads + kv) * d].view(T, kv, d), pos, theta)
    wv = x[:, (heads + kv) * d:].view(T, kv, d)
    assert rel_err(q, wq) < tol(dtype)
    want_k, want_v = torch.zeros(pages, kv, page, d, dtype=torch.float64), torch.zeros(pages, kv, d, page, dtype=torch.float64)
    for t, slot in enumerate(slot_list):
        if slot >= 0:
            want_k[slot // page, :, slot % page, :] = wk[t]
            want_v[slot // page, :, :, slot % page] = wv[t]
    assert rel_err(kc, want_k) < tol(dtype) and rel_err(vc, want_v) < tol(dtype)
    untouched = want_v == 0
    assert float(vc.double().cpu()[untouched].abs().sum()) == 0  # nothing else was written


@pytest.mark.parametrize("T,H,heads,kv,d,page,bias", [(1, 64, 4, 2, 32, 16, True), (8, 2048, 16, 16, 128, 16, True),
                                                       (16, 96, 3, 1, 32, 32, False), (5, 72, 6, 3, 64, 16, True),
                                                       (3, 1160, 5, 5, 96, 16, True), (9, 904, 2, 1, 128, 64, False),
                                                       (17, 96, 3, 1, 32, 16, True), (32, 2048, 16, 16, 128, 16, True),
                                                       (29, 904, 7, 1, 64, 32, False)])
def test_qkv_rope_skinny_equals_product_then_epilogue(T, H, heads, kv, d, page, bias):
    """The one-launch q/k/v path for few tokens writes what the product followed by qkv_rope_append writes."""
    from inferx_amd import ops
    from inferx_amd.parts.rope import Rotary
    dt = torch.bfloat16
    width = (heads + 2 * kv) * d
    x, w = rnd(T, H, dtype=dt), rnd(width, H, seed=1, dtype=dt, scale=H ** -0.5)
    b = rnd(width, seed=2, dtype=dt) if bias else None
    pos = torch.arange(40, 40 + T, dtype=torch.int32, device=DEV)
    slots = (torch.arange(T, dtype=torch.int32, device=DEV) * 3 + 5)
    table = torch.empty(T, d // 2, 2, device=DEV)
    ops.rope_table(table, pos, Rotary(1e6, d).frequencies().to(DEV))
    pages = 6
    outs = []
    for fused in (False, True):
        q = torch.full((T, heads, d), float("nan"), dtype=dt, device=DEV)
        kc = torch.zeros(pages, kv, page, d, dtype=dt, device=DEV)
        vc = torch.zeros(pages, kv, d, page, dtype=dt, device=DEV)
        if fused:
            ops.qkv_rope_skinny(x, w, b, table, slots, q, kc, vc, heads, kv, d)
        else:
            ops.qkv_rope_append(torch.matmul(x, w.t()), b, table, slots, q, kc, vc, heads, kv, d)
        outs.append((q, kc, vc))
    for a, c in zip(outs[0], outs[1]):
        assert rel_err(c, a) < 1e-2  # the two products round differently in the last bit of bfloat16
    # and against float64 from the start
    xd = x.double().cpu() @ w.double().cpu().T + (b.double().cpu() if bias else 0)
    wq = pm.apply_rope(xd[:, :heads * d].view(T, heads, d), pos.cpu(), 1e6)
    assert rel_err(outs[1][0], wq) < 1.5e-2


def test_argmax_first_maximum():
    # reference vector: tests/unit/host_sampling_test.cc:12-17 ({1, 4, 2} -> 1); ties go to the lowest index
    from inferx_amd import ops
    logits = torch.tensor([[1.0, 4.0, 2.0], [3.0, 3.0, 1.0], [-1.0, -5.0, -1.0]], device=DEV)
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out)
    assert out.tolist() == [1, 0, 0]
    big = rnd(4, 151936, seed=3)
    big[2, 77777] = 50.0
    big[2, 150000] = 50.0
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.argmax(big, out)
    assert out.tolist() == [int(r.argmax()) for r in big.cpu()[:2]] + [77777, int(big[3].argmax())]


def draw(logits, temperature, top_k=0, top_p=1.0, min_p=0.0, seed=0, counter=0):
    from inferx_amd import ops
    R = logits.shape[0]
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    f = lambda v, dt: torch.full((R,), v, dtype=dt, device=DEV)
    ops.sample(logits, out, f(temperature, torch.float32), f(top_p, torch.float32), f(top_k, torch.int32),
               f(min_p, torch.float32), f(seed, torch.int64), f(counter, torch.int64))
    return out.tolist()


def test_deterministic_settings_equal_argmax():
    # reference: tests/kernel/sampling_test.cc:213-364 (t = 0, top_k = 1, min_p = 1, a dominant nucleus)
    logits = rnd(6, 1000, seed=5, scale=2.0)
    want = logits.argmax(-1).tolist()
    assert draw(logits, 0.0) == want
    assert draw(logits, 0.7, top_k=1) == want
    assert draw(logits, 0.7, min_p=1.0) == want
    peaked = logits.clone()
    peaked[torch.arange(6), torch.tensor(want)] += 30.0
    assert draw(peaked, 1.0, top_p=0.5) == want


@pytest.mark.parametrize("settings", [dict(top_k=5), dict(top_p=0.6), dict(min_p=0.2), dict(top_k=8, top_p=0.8),
                                      dict()])
def test_random_settings_stay_in_the_support_and_repeat(settings):
    # reference: sampling_test.cc:265-291, 366-438; tests/unit/host_sampling_test.cc:34-53
    logits = rnd(1, 300, seed=6, scale=2.5)
    support = set(pm.sampling_support(logits[0].cpu(), 0.8, **settings))
    seen = set()
    for seed in range(40):
        a = draw(logits, 0.8, seed=seed, counter=3, **settings)
        assert a == draw(logits, 0.8, seed=seed, counter=3, **settings)  # a pinned seed reproduces
        assert a[0] in support
        seen.add(a[0])
    assert len(seen) > 1 or len(support) == 1
    assert len({draw(logits, 0.8, seed=1, counter=c, **settings)[0] for c in range(40)}) > 1 or len(support) == 1


@pytest.mark.parametrize("settings", [dict(top_k=40), dict(top_p=0.9), dict(top_k=500, top_p=0.95, min_p=0.001),
                                      dict(min_p=0.05), dict(top_k=100000)])
@pytest.mark.parametrize("spread", [3.0, 1e-3])
def test_cut_offs_on_a_real_vocabulary(settings, spread):
    """151,936 logits, broad (the boundary's bin of the first histogram is small) and nearly uniform (all tokens
    fall into one or two bins, which are cut finer twice): every draw lies in the plain implementation's support,
    and with many seeds the draws reach beyond the most probable tokens."""
    V = 151936
    logits = rnd(2, V, seed=11, scale=spread)
    supports = [set(pm.sampling_support(logits[r].cpu(), 0.8, **settings)) for r in range(2)]
    seen = [set(), set()]
    for seed in range(24):
        got = draw(logits, 0.8, seed=seed, counter=seed * 7, **settings)
        assert got == draw(logits, 0.8, seed=seed, counter=seed * 7, **settings)
        for r in range(2):
            assert got[r] in supports[r], (settings, spread, seed, r, got[r], len(supports[r]))
            seen[r].add(got[r])
    assert all(len(s) > 3 for s in seen)


def test_cut_offs_with_many_equal_logits():
    """Three distinct values, tens of thousands of tokens each: tokens that cannot be told apart stay together, so
    the support is every token at least as probable as the boundary token (the plain implementation cuts the ties
    by index)."""
    V = 90000
    logits = torch.full((1, V), -2.0, device=DEV)
    logits[0, 1::3] = 1.0
    logits[0, 2::3] = 0.5
    exact = set(pm.sampling_support(logits[0].cpu(), 1.0, top_k=40000))
    with_ties = set(range(1, V, 3)) | set(range(2, V, 3))  # 30,000 + 30,000: the boundary lies among the second value
    assert exact < with_ties
    seen = set()
    for seed in range(30):
        tok = draw(logits, 1.0, top_k=40000, seed=seed)[0]
        assert tok in with_ties
        seen.add(tok % 3)
    assert seen == {1, 2}
    for seed in range(10):
        assert draw(logits, 1.0, top_k=2000, seed=seed)[0] % 3 == 1  # the rank falls among the first value's tokens
    # up to 2,048 equal tokens are ranked exactly, by index like the plain implementation
    few = torch.full((1, 5000), -3.0, device=DEV)
    few[0, 7::5] = 2.0  # 999 tokens tied at the top
    exact = set(pm.sampling_support(few[0].cpu(), 1.0, top_k=300))
    assert exact == set(range(7, 7 + 5 * 300, 5))
    seen = {draw(few, 1.0, top_k=300, seed=seed)[0] for seed in range(60)}
    assert seen <= exact and len(seen) > 20


def test_sampling_follows_the_distribution():
    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0]], device=DEV)
    p = torch.softmax(logits[0].cpu().double() / 0.9, -1)
    n = 4000
    counts = torch.zeros(4)
    for seed in range(n):
        counts[draw(logits, 0.9, seed=seed)[0]] += 1
    assert float((counts / n - p).abs().max()) < 0.03


def test_logprobs():
    # reference vector: tests/unit/host_sampling_test.cc:55-69 (logits {0, 1, 2}, top 2 -> ids {2, 1})
    from inferx_amd import ops
    logits = torch.tensor([[0.0, 1.0, 2.0], [3.0, 3.0, -1.0]], device=DEV)
    chosen = torch.tensor([2, 1], dtype=torch.int32, device=DEV)
    lp, ids, tlp = torch.empty(2, device=DEV), torch.empty(2, 2, dtype=torch.int32, device=DEV), torch.empty(2, 2, device=DEV)
    ops.logprobs(logits, chosen, lp, ids, tlp)
    log_z = math.log(math.exp(0) + math.exp(1) + math.exp(2))
    assert abs(float(lp[0]) - (2 - log_z)) < 1e-6
    assert ids.tolist() == [[2, 1], [0, 1]]  # equal logits: the lower index first
    assert abs(float(tlp[0, 0]) - (2 - log_z)) < 1e-6 and abs(float(tlp[0, 1]) - (1 - log_z)) < 1e-6
    big = rnd(3, 151936, seed=9, scale=3.0)
    chosen = torch.tensor([5, 77777, 151935], dtype=torch.int32, device=DEV)
    lp, ids, tlp = torch.empty(3, device=DEV), torch.empty(3, 5, dtype=torch.int32, device=DEV), torch.empty(3, 5, device=DEV)
    ops.logprobs(big, chosen, lp, ids, tlp)
    want = torch.log_softmax(big.double().cpu(), -1)
    top = torch.topk(want, 5, dim=-1)
    assert ids.cpu().long().tolist() == top.indices.tolist()
    assert float((tlp.cpu().double() - top.values).abs().max()) < 1e-4
    assert float((lp.cpu().double() - want[torch.arange(3), chosen.cpu().long()]).abs().max()) < 1e-4


def test_penalties_and_masks():
    # reference vector: tests/unit/host_sampling_test.cc:19-32 ({5, 4, 3}, presence 3 on id 0, mask on id 1 -> 2)
    from inferx_amd import ops
    logits = torch.tensor([[5.0, 4.0, 3.0], [2.0, -2.0, 1.0]], device=DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    f32 = lambda v: torch.tensor(v, dtype=torch.float32, device=DEV)
    ops.apply_penalties(logits, i32([0, 1, 3]), i32([0, 0, 1]), i32([1, 2, 1]), f32([3.0, 0.5]), f32([0.0, 0.25]),
                        f32([1.0, 2.0]), i32([0, 1, 1]), i32([1]))
    want = [[5.0 - 3.0, -math.inf, 3.0], [2.0 / 2 - 0.5 - 0.5, -2.0 * 2 - 0.5 - 0.25, 1.0]]
    assert logits.cpu().tolist() == want
    out = torch.empty(2, dtype=torch.int32, device=DEV)
    ops.argmax(logits, out)
    assert out.tolist()[0] == 2


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,N,K", [(33, 2048, 2048), (300, 1000, 136), (512, 6144, 2048), (64, 131, 100), (1, 17, 16),
                                   (200, 5003, 72), (2048, 2048, 5632)])
def test_library_product(T, N, K, out_dtype):
    """The vendor library's dense product through its C interface: right, or refused with nothing written."""
    from inferx_amd import ops
    x, w = rnd(T, K, dtype=torch.bfloat16), rnd(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    out = torch.full((T, N), 7.0, dtype=out_dtype, device=DEV)
    if not ops.gemm_bf16(x, w, out):
        torch.cuda.synchronize()
        assert bool((out == 7.0).all()), "a refused product must not write"
        assert not ops.gemm_bf16(x, w, out)  # and stays refused
        return
    want = x.double().cpu() @ w.double().cpu().T
    assert rel_err(out, want) < (1e-5 if out_dtype == torch.float32 else 8e-3)


def test_library_product_in_a_graph_and_on_two_streams():
    """Replays of a captured product follow their inputs; products on two streams at once keep to their own
    workspaces (a shape whose kernel splits the reduction and sums the parts through the workspace)."""
    from inferx_amd import ops
    T, N, K = 48, 2048, 5632
    w = rnd(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    x = rnd(T, K, dtype=torch.bfloat16)
    out = torch.empty(T, N, dtype=torch.bfloat16, device=DEV)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        assert ops.gemm_bf16(x, w, out)  # the stream's first product, not recorded: it allocates the workspace
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        ops.gemm_bf16(x, w, out)
    for seed in (3, 4, 5):
        x.copy_(rnd(T, K, seed=seed, dtype=torch.bfloat16))
        g.replay()
        torch.cuda.synchronize()
        eager = torch.empty_like(out)
        assert ops.gemm_bf16(x, w, eager)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay with seed {seed} differs from the eager product"
        assert rel_err(out, x.double().cpu() @ w.double().cpu().T) < 8e-3
    # two streams at once, many products each
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    xa, xb = rnd(T, K, seed=8, dtype=torch.bfloat16), rnd(T, K, seed=9, dtype=torch.bfloat16)
    oa, ob = [torch.empty_like(out) for _ in range(20)], [torch.empty_like(out) for _ in range(20)]
    torch.cuda.synchronize()
    for i in range(20):
        with torch.cuda.stream(a):
            ops.gemm_bf16(xa, w, oa[i])
        with torch.cuda.stream(b):
            ops.gemm_bf16(xb, w, ob[i])
    torch.cuda.synchronize()
    assert all(torch.equal(o, oa[0]) for o in oa) and all(torch.equal(o, ob[0]) for o in ob)
    assert rel_err(oa[0], xa.double().cpu() @ w.double().cpu().T) < 8e-3
    assert rel_err(ob[0], xb.double().cpu() @ w.double().cpu().T) < 8e-3


def test_the_probes_of_the_machine_s_ceilings():
    """The two probes that the benchmark prices its results against: a pure read and pure matrix-core products.
    Their figures are rates, so only their sanity is checked: positive, finite, and within what one MI355X can do."""
    import math
    from inferx_amd import ops
    got = ops.measured_ceilings(DEV, read_bytes=1 << 30)
    read, mfma = got["hbm_read_gbs"], got["mfma_bf16_tflops"]
    assert math.isfinite(read) and 200.0 < read < 30000.0
    assert math.isfinite(mfma) and 50.0 < mfma < 5200.0


def test_random_weights_are_the_same_bits_on_the_host_and_on_the_device():
    """The weights that a benchmark draws on the device can be drawn again on the host: element i of a tensor is a
    function of (seed, name, i) in integer arithmetic."""
    from inferx_amd.weights.random_init import counter_normal
    for shape, std in (((60, 1408, 64), 0.02), ((3, 17), 1.0), (((1 << 24) + 5,), 0.5)):
        host = counter_normal(11, "model.layers.2.mlp.experts.5.up_proj.weight", shape, std)
        device = counter_normal(11, "model.layers.2.mlp.experts.5.up_proj.weight", shape, std, device="cuda:0")
        assert torch.equal(host, device.cpu())
