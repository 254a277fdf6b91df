"""The mixture-of-experts kernels alone against PyTorch references: router, grouping,
grouped products (plain and matrix-core), combine.  Properties follow the reference's
tests/kernel/moe_test.cc (lines cited per test)."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rnd(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def rel_err(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max()) / max(float(want.abs().max()), 1e-30)


def route_reference(x, wr, k, renorm, scale=1.0):
    p = torch.softmax(x.double().cpu() @ wr.double().cpu().T, -1)
    w, e = torch.topk(p, k, dim=-1)
    if renorm:
        w = w / w.sum(-1, keepdim=True)
    return w * scale, e


@pytest.mark.parametrize("T,H,E,k,renorm", [(24, 64, 8, 2, False), (7, 200, 60, 4, True), (130, 72, 5, 1, False),
                                            (3, 2048, 64, 8, True), (50, 96, 32, 32, True),
                                            (300, 136, 60, 4, True), (203, 40, 70, 6, False)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_route(T, H, E, k, renorm, dtype):
    # reference: moe_test.cc:170-246 (router equals host to 1e-5, renormalised sums to 1, un-normalised below)
    from inferx_amd import ops
    x, wr, wsg = rnd(T, H, dtype=dtype), rnd(E, H, seed=1, dtype=dtype, scale=0.3), rnd(1, H, seed=2, dtype=dtype, scale=0.1)
    topk_w = torch.empty(T, k, dtype=torch.float32, device=DEV)
    topk_e = torch.empty(T, k, dtype=torch.int32, device=DEV)
    gate = torch.empty(T, dtype=torch.float32, device=DEV)
    ops.moe_route(x, wr, wsg, topk_w, topk_e, gate, renorm, 1.0)
    want_w, want_e = route_reference(x, wr, k, renorm)
    assert torch.equal(topk_e.cpu().long(), want_e)
    assert rel_err(topk_w, want_w) < 1e-5
    assert rel_err(gate, torch.sigmoid(x.double().cpu() @ wsg.double().cpu().T)[:, 0]) < 1e-5
    sums = topk_w.sum(-1).cpu()
    if renorm:
        assert torch.allclose(sums, torch.ones(T), atol=1e-5)
    elif k < E:
        assert (sums < 0.9999).all()


def test_route_refuses_what_it_cannot_do():
    from inferx_amd import ops
    x, wr = rnd(4, 96), rnd(40, 96, seed=1)
    with pytest.raises(ops.KernelError, match="top_k"):
        ops.moe_route(x, wr, None, torch.empty(4, 33, device=DEV), torch.empty(4, 33, dtype=torch.int32, device=DEV),
                      None, False, 1.0)


def test_route_equal_logits_take_the_lowest_indices():
    # reference vector: moe_test.cc:248-273
    from inferx_amd import ops
    T, H, E, k = 5, 16, 32, 2
    x = torch.ones(T, H, device=DEV)
    wr = torch.full((E, H), 0.25 / H, device=DEV)
    topk_w = torch.empty(T, k, device=DEV)
    topk_e = torch.empty(T, k, dtype=torch.int32, device=DEV)
    ops.moe_route(x, wr, None, topk_w, topk_e, None, False, 1.0)
    assert topk_e.cpu().tolist() == [[0, 1]] * T
    assert torch.allclose(topk_w.cpu(), torch.full((T, k), 1 / 32))


def dispatch(topk_e, E, tile_rows=0):
    from inferx_amd import ops
    T, k = topk_e.shape
    A = T * k
    offsets = torch.empty(E + 1, dtype=torch.int32, device=DEV)
    rows = torch.empty(A, dtype=torch.int32, device=DEV)
    dest = torch.empty(A, dtype=torch.int32, device=DEV)
    tile_map = None
    if tile_rows:
        tile_map = torch.full((2 * ops.moe_max_tiles(A, E, tile_rows) + 1,), -7, dtype=torch.int32, device=DEV)
    ops.moe_dispatch(topk_e, offsets, rows, dest, E, tile_rows, tile_map)
    return offsets, rows, dest, tile_map


@pytest.mark.parametrize("T,E,k,tile_rows", [(24, 8, 2, 16), (300, 60, 4, 32), (1, 4, 2, 16), (1000, 7, 3, 64),
                                             (40, 64, 1, 0), (2048, 60, 4, 160), (3000, 60, 4, 160), (500, 200, 3, 32),
                                             (600, 1024, 2, 16), (4100, 3, 2, 0)])
def test_dispatch_is_a_stable_bijection(T, E, k, tile_rows):
    # reference: moe_test.cc:277-350
    g = torch.Generator().manual_seed(T)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if E > 3:
        topk_e[topk_e == 2] = 3  # expert 2 stays empty (an assignment may then repeat expert 3; fine for grouping)
    offsets, rows, dest, tile_map = dispatch(topk_e.to(DEV), E, tile_rows)
    offsets, rows, dest = offsets.cpu(), rows.cpu(), dest.cpu()
    flat = topk_e.flatten()
    A = T * k
    assert offsets[0] == 0 and offsets[E] == A
    assert sorted(dest.tolist()) == list(range(A))  # every assignment exactly once
    for a in range(A):
        e = int(flat[a])
        assert offsets[e] <= dest[a] < offsets[e + 1]      # in its expert's range
        assert rows[dest[a]] == a // k                      # rows and dest are inverse
    if E > 3:
        assert offsets[2] == offsets[3]                     # an empty expert has an empty range
    for e in range(E):
        mine = [int(dest[a]) for a in range(A) if int(flat[a]) == e]
        assert mine == sorted(mine)                         # stable: assignment order is kept
    if tile_rows:
        mt = (tile_map.numel() - 1) // 2
        n = int(tile_map[2 * mt])
        te, tr = tile_map[:n].cpu().tolist(), tile_map[mt:mt + n].cpu().tolist()
        covered = []
        for e_, r0 in zip(te, tr):
            assert offsets[e_] <= r0 < offsets[e_ + 1]
            covered += list(range(r0, min(r0 + tile_rows, int(offsets[e_ + 1]))))
        assert covered == list(range(A))  # tiles cover every row once, in order


@pytest.mark.parametrize("T,H,E,k,renorm,tile_rows", [(1, 64, 4, 2, False, 16), (8, 2048, 60, 4, False, 16),
                                                       (11, 96, 8, 3, True, 32), (16, 72, 5, 1, False, 0),
                                                       (16, 200, 256, 32, True, 16), (16, 136, 60, 4, True, 16),
                                                       (5, 88, 7, 3, False, 0), (13, 200, 256, 8, True, 16),
                                                       # at most 64 assignments: experts with more rows than a tile; 256 experts
                                                       (16, 64, 3, 2, False, 4), (4, 200, 256, 8, True, 16), (7, 80, 130, 9, False, 2),
                                                       # one token, also with 64 and 65 router rows and a wide row
                                                       (1, 2048, 60, 4, False, 16), (1, 200, 63, 8, True, 16), (1, 96, 64, 3, False, 16),
                                                       (1, 4104, 17, 5, True, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_route_and_dispatch_for_few_tokens(T, H, E, k, renorm, tile_rows, dtype):
    """Scores, selection and grouping in one launch (up to 16 tokens) give exactly what the separate kernels give."""
    from inferx_amd import ops
    x, wr, wsg = rnd(T, H, dtype=dtype), rnd(E, H, seed=1, dtype=dtype, scale=0.3), rnd(1, H, seed=2, dtype=dtype, scale=0.1)
    A = T * k
    mk = lambda *shape, dt=torch.int32: torch.full(shape, -9, dtype=dt, device=DEV)
    w1, e1, g1 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
    ops.moe_route(x, wr, wsg, w1, e1, g1, renorm, 1.0)
    o1, r1, d1, tm1 = dispatch(e1, E, tile_rows)
    w2, e2, g2 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
    o2, r2, d2 = mk(E + 1), mk(A), mk(A)
    tm2 = mk(2 * ops.moe_max_tiles(A, E, tile_rows) + 1) if tile_rows else None
    ops.moe_route_dispatch(x, wr, wsg, w2, e2, g2, renorm, 1.0, o2, r2, d2, tile_rows, tm2)
    assert torch.equal(e1, e2) and torch.equal(o1, o2) and torch.equal(r1, r2) and torch.equal(d1, d2)
    assert rel_err(w2, w1) < 1e-6 and rel_err(g2, g1) < 1e-6
    if tile_rows:
        mt = (tm1.numel() - 1) // 2
        n = int(tm1[2 * mt])
        assert int(tm2[2 * mt]) == n and torch.equal(tm1[:n], tm2[:n]) and torch.equal(tm1[mt:mt + n], tm2[mt:mt + n])


def test_route_in_one_launch_again_and_again():
    """The one-launch router counts its workgroups off on a counter that every launch leaves at zero, and its
    last workgroup reads what workgroups on other dies wrote: many launches of changing sizes one after the
    other, without waiting, all agree with the separate kernels."""
    from inferx_amd import ops
    mk = lambda *shape, dt=torch.int32: torch.full(shape, -9, dtype=dt, device=DEV)
    cases, got = [(3, 2048, 60, 4), (16, 136, 60, 4), (1, 64, 4, 2), (9, 200, 256, 8), (8, 2048, 60, 4)] * 40, []
    for i, (T, H, E, k) in enumerate(cases):
        x, wr, wsg = (rnd(T, H, seed=i, dtype=torch.bfloat16), rnd(E, H, seed=100 + i, dtype=torch.bfloat16, scale=0.3),
                      rnd(1, H, seed=200 + i, dtype=torch.bfloat16, scale=0.1))
        w2, e2, g2 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
        o2, r2, d2 = mk(E + 1), mk(T * k), mk(T * k)
        ops.moe_route_dispatch(x, wr, wsg, w2, e2, g2, True, 1.0, o2, r2, d2, 0, None)
        got.append((x, wr, wsg, w2, e2, g2, o2, r2, d2))
    for (T, H, E, k), (x, wr, wsg, w2, e2, g2, o2, r2, d2) in zip(cases, got):
        w1, e1, g1 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
        ops.moe_route(x, wr, wsg, w1, e1, g1, True, 1.0)
        o1, r1, d1, _ = dispatch(e1, E, 0)
        assert torch.equal(e1, e2) and torch.equal(o1, o2) and torch.equal(r1, r2) and torch.equal(d1, d2)
        assert rel_err(w2, w1) < 1e-6 and rel_err(g2, g1) < 1e-6


def grouped_reference(a, w, offsets, rows, gate_up):
    a, w = a.double().cpu(), w.double().cpu()
    E = w.shape[0]
    A = int(offsets[E])
    n = w.shape[1] // 2 if gate_up else w.shape[1]
    out = torch.zeros(A, n, dtype=torch.float64)
    for e in range(E):
        for r in range(int(offsets[e]), int(offsets[e + 1])):
            x = a[int(rows[r])] if rows is not None else a[r]
            z = w[e] @ x
            out[r] = torch.nn.functional.silu(z[:n]) * z[n:] if gate_up else z
    return out


GROUPED = [(24, 64, 8, 2, 32), (300, 96, 8, 3, 48), (9, 72, 5, 1, 40), (700, 256, 60, 4, 176), (3, 2048, 60, 4, 1408),
           (20, 1160, 5, 2, 200)]


@pytest.mark.parametrize("T,H,E,k,mi", GROUPED)
@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
def test_grouped_plain(T, H, E, k, mi, dtype, wdtype):
    from inferx_amd import ops
    if T * mi * H > 300 * 96 * 48 * 40:
        pytest.skip("large for the plain kernel's test")
    g = torch.Generator().manual_seed(1)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, rows, dest, _ = dispatch(topk_e, E)
    x = rnd(T, H, dtype=dtype)
    w13, w2 = rnd(E, 2 * mi, H, seed=2, dtype=wdtype, scale=H ** -0.5), rnd(E, H, mi, seed=3, dtype=wdtype, scale=mi ** -0.5)
    act = torch.empty(T * k, mi, dtype=dtype, device=DEV)
    ops.moe_grouped_plain(x, w13, act, offsets, rows, True)
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    assert rel_err(act, grouped_reference(x, w13, offsets.cpu(), rows.cpu(), True)) < tol
    y = torch.empty(T * k, H, dtype=dtype, device=DEV)
    ops.moe_grouped_plain(act, w2, y, offsets, None, False)
    assert rel_err(y, grouped_reference(act, w2, offsets.cpu(), None, False)) < tol


@pytest.mark.parametrize("T,H,E,k,mi", GROUPED)
@pytest.mark.parametrize("tile_rows", [16, 32, 64])
@pytest.mark.parametrize("k_split", [1, 4])
def test_grouped_mfma(T, H, E, k, mi, tile_rows, k_split):
    from inferx_amd import ops
    g = torch.Generator().manual_seed(1)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, rows, dest, tile_map = dispatch(topk_e, E, tile_rows)
    x = rnd(T, H, dtype=torch.bfloat16)
    w13 = rnd(E, 2 * mi, H, seed=2, dtype=torch.bfloat16, scale=H ** -0.5)
    w2 = rnd(E, H, mi, seed=3, dtype=torch.bfloat16, scale=mi ** -0.5)
    act = torch.full((T * k, mi), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.moe_grouped_mfma(x, w13, act, offsets, rows, tile_map, tile_rows, True, k_split)
    assert rel_err(act, grouped_reference(x, w13, offsets.cpu(), rows.cpu(), True)) < 1.5e-2
    y = torch.full((T * k, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.moe_grouped_mfma(act, w2, y, offsets, None, tile_map, tile_rows, False, k_split)
    assert rel_err(y, grouped_reference(act, w2, offsets.cpu(), None, False)) < 1.5e-2
    # bitwise repeatable (reference: moe_test.cc:972-1046)
    y2 = torch.empty_like(y)
    ops.moe_grouped_mfma(act, w2, y2, offsets, None, tile_map, tile_rows, False, k_split)
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


@pytest.mark.parametrize("wide", [False, True])
@pytest.mark.parametrize("T,H,E,k,mi", GROUPED + [(900, 136, 6, 2, 88), (2048, 512, 12, 4, 352)])
def test_grouped_tiled(T, H, E, k, mi, wide):
    """Experts with a handful of rows, with about one tile of them, and with several tiles (the last one partial);
    128 and 256 weight rows per workgroup, which give the same bits."""
    from inferx_amd import ops
    g = torch.Generator().manual_seed(1)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, rows, dest, tile_map = dispatch(topk_e, E, ops.moe_tiled_rows(wide))  # tiles of 160 rows, wide 192
    x = rnd(T, H, dtype=torch.bfloat16)
    w13 = rnd(E, 2 * mi, H, seed=2, dtype=torch.bfloat16, scale=H ** -0.5)
    w2 = rnd(E, H, mi, seed=3, dtype=torch.bfloat16, scale=mi ** -0.5)
    act = torch.full((T * k, mi), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.moe_grouped_tiled(x, w13, act, offsets, rows, tile_map, True, wide)
    y = torch.full((T * k, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.moe_grouped_tiled(act, w2, y, offsets, None, tile_map, False, wide)
    if wide:
        _, _, _, narrow_map = dispatch(topk_e, E, ops.moe_tiled_rows(False))
        act_n, y_n = torch.empty_like(act), torch.empty_like(y)
        ops.moe_grouped_tiled(x, w13, act_n, offsets, rows, narrow_map, True, False)
        ops.moe_grouped_tiled(act, w2, y_n, offsets, None, narrow_map, False, False)
        if H % 512 and mi % 512:
            # the same sums in the same order (rows of a multiple of 1,024 bytes start the reduction at a stage
            # that depends on the tile, and the two forms cut tiles differently)
            assert torch.equal(act.view(torch.int16), act_n.view(torch.int16))
            assert torch.equal(y.view(torch.int16), y_n.view(torch.int16))
        else:
            assert rel_err(act, act_n) < 1e-2 and rel_err(y, y_n) < 1e-2
    if T <= 900:
        assert rel_err(act, grouped_reference(x, w13, offsets.cpu(), rows.cpu(), True)) < 1.5e-2
        assert rel_err(y, grouped_reference(act, w2, offsets.cpu(), None, False)) < 1.5e-2
    else:  # large: against the wavefront-level kernel, which the small cases pin to the reference
        act2, y2 = torch.empty_like(act), torch.empty_like(y)
        _, _, _, map64 = dispatch(topk_e, E, 64)
        ops.moe_grouped_mfma(x, w13, act2, offsets, rows, map64, 64, True, 1)
        ops.moe_grouped_mfma(act, w2, y2, offsets, None, map64, 64, False, 1)
        assert rel_err(act, act2) < 1e-2 and rel_err(y, y2) < 1e-2


@pytest.mark.parametrize("T,N,K", [(3, 40, 264), (16, 33, 1160), (2, 16, 8), (5, 48, 520)])
def test_streaming_kernels_read_nothing_past_their_operands(T, N, K):
    """Reduction widths that leave a wavefront a ragged last round: what lies behind the last row of the weights
    and of the activations (here NaN) must not reach a result, not even multiplied by zero."""
    from inferx_amd import ops
    xbuf = torch.full((T + 1, K), float("nan"), dtype=torch.bfloat16, device=DEV)
    wbuf = torch.full((2 * N + 1, K), float("nan"), dtype=torch.bfloat16, device=DEV)
    xbuf[:T] = rnd(T, K, dtype=torch.bfloat16)
    wbuf[:2 * N] = rnd(2 * N, K, seed=1, dtype=torch.bfloat16, scale=K ** -0.5)
    x, w = xbuf[:T], wbuf[:N]
    out = torch.full((T, N), float("nan"), device=DEV)
    ops.linear_skinny_f32(x, w, out)
    want = x.double().cpu() @ w.double().cpu().t()
    assert torch.isfinite(out).all() and rel_err(out, want) < 1e-5
    # the grouped product, one expert: gate|up over both halves of the weights, then a plain product
    offsets = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    tile_map = torch.tensor([0, 0, 0, 0, 1], dtype=torch.int32, device=DEV)  # one tile of expert 0 from row 0
    for k_split in (1, 4):
        act = torch.full((T, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.moe_grouped_mfma(x, wbuf[:2 * N].unsqueeze(0), act, offsets, None, tile_map, 16, True, k_split)
        z = x.double().cpu() @ wbuf[:2 * N].double().cpu().t()
        assert torch.isfinite(act).all()
        assert rel_err(act, torch.nn.functional.silu(z[:, :N]) * z[:, N:]) < 1.5e-2
        y = torch.full((T, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.moe_grouped_mfma(x, w.unsqueeze(0), y, offsets, None, tile_map, 16, False, k_split)
        assert torch.isfinite(y).all() and rel_err(y, want) < 1.5e-2


@pytest.mark.parametrize("T,N,K", [(1, 301, 72), (8, 151936, 2048), (16, 384, 96), (33, 1000, 64), (64, 256, 40)])
def test_linear_skinny_f32(T, N, K):
    from inferx_amd import ops
    x, w = rnd(T, K, dtype=torch.bfloat16), rnd(N, K, seed=1, dtype=torch.bfloat16, scale=K ** -0.5)
    out = torch.full((T, N), float("nan"), device=DEV)
    ops.linear_skinny_f32(x, w, out)
    assert rel_err(out, x.double().cpu() @ w.double().cpu().T) < 1e-5  # float32 accumulation of exact products


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gather_then_combine_is_the_identity(dtype):
    # reference: moe_test.cc:352-411 (weights 0.25 / 0.75)
    from inferx_amd import ops
    T, H, E, k = 24, 64, 8, 2
    g = torch.Generator().manual_seed(2)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    offsets, rows, dest, _ = dispatch(topk_e, E)
    x = rnd(T, H, dtype=dtype)
    y = x[rows.long()]  # what an identity expert would produce
    topk_w = torch.tensor([[0.25, 0.75]] * T, device=DEV)
    out = torch.empty_like(x)
    ops.moe_combine(y, dest, topk_w, None, None, out)
    assert rel_err(out, x) < (1e-6 if dtype == torch.float32 else 1e-2)
    shared, gate = rnd(T, H, seed=5, dtype=dtype), torch.rand(T, device=DEV)
    ops.moe_combine(y, dest, topk_w, shared, gate, out)
    assert rel_err(out, x.double() + gate.double()[:, None] * shared.double()) < (1e-6 if dtype == torch.float32 else 1e-2)
    ops.moe_combine(y, dest, topk_w, shared, None, out)  # an ungated shared expert adds exactly its output
    assert rel_err(out, x.double() + shared.double()) < (1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("T,H,E,k", [(1, 64, 4, 2), (8, 2048, 60, 4), (16, 136, 60, 4), (5, 88, 7, 3), (13, 200, 256, 8),
                                     (1, 2048, 60, 4), (1, 200, 63, 8), (1, 96, 64, 3), (1, 4104, 17, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_route_and_dispatch_in_one_launch(T, H, E, k, dtype):
    """The norm before the feed-forward as part of the one-launch router: the residual stream is brought up to
    date exactly, the normalised rows are those of the separate norm kernel up to the rounding of one sum, and
    the routing is exactly that of the separate kernels on the rows it wrote."""
    from inferx_amd import ops
    mk = lambda *shape, dt=torch.int32: torch.full(shape, -9, dtype=dt, device=DEV)
    h0, delta = rnd(T, H, seed=3, dtype=torch.float32, scale=2.0), rnd(T, H, seed=4, dtype=dtype)
    gamma = (1.0 + rnd(H, seed=5, dtype=torch.float32, scale=0.2)).to(dtype)
    wr, wsg = rnd(E, H, seed=1, dtype=dtype, scale=0.3), rnd(1, H, seed=2, dtype=dtype, scale=0.1)
    eps = 1e-5
    h1, x1 = h0.clone(), torch.empty(T, H, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h1, delta, gamma, x1, eps)
    for tile_rows in (0, 16):
        h2, x2 = h0.clone(), torch.full((T, H), 7.0, dtype=dtype, device=DEV)
        w2, e2, g2 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
        o2, r2, d2 = mk(E + 1), mk(T * k), mk(T * k)
        tm2 = mk(2 * ops.moe_max_tiles(T * k, E, tile_rows) + 1) if tile_rows else None
        ops.moe_route_dispatch(None, wr, wsg, w2, e2, g2, True, 1.0, o2, r2, d2, tile_rows, tm2,
                               norm=(h2, delta, gamma, eps, x2))
        assert torch.equal(h2, h1)
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -21
        assert ((x2.float() - x1.float()).abs() <= ulp * x1.float().abs() + 1e-30).all()
        w1, e1, g1 = mk(T, k, dt=torch.float32), mk(T, k), mk(T, dt=torch.float32)
        ops.moe_route(x2, wr, wsg, w1, e1, g1, True, 1.0)
        o1, r1, d1, tm1 = dispatch(e1, E, tile_rows)
        assert torch.equal(e1, e2) and torch.equal(o1, o2) and torch.equal(r1, r2) and torch.equal(d1, d2)
        assert rel_err(w2, w1) < 1e-6 and rel_err(g2, g1) < 1e-6


@pytest.mark.parametrize("T,H,E,k,mi,S", [(1, 64, 4, 2, 32, 48), (8, 2048, 60, 4, 1408, 5632), (16, 136, 60, 4, 40, 24),
                                          (21, 96, 8, 3, 48, 80), (40, 72, 5, 1, 40, 200), (64, 264, 7, 2, 88, 1000)])
def test_routed_and_shared_experts_in_one_launch(T, H, E, k, mi, S):
    """The launch that holds the routed experts' product and the shared expert's: the routed part is bit for bit
    the routed launch's, the shared part is the product of all tokens with the shared weights; both products
    (gate|up with SwiGLU, down), every tile height that takes the token count."""
    from inferx_amd import ops
    g = torch.Generator().manual_seed(1)
    topk_e = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    x = rnd(T, H, dtype=torch.bfloat16)
    w13 = rnd(E, 2 * mi, H, seed=2, dtype=torch.bfloat16, scale=H ** -0.5)
    w2 = rnd(E, H, mi, seed=3, dtype=torch.bfloat16, scale=mi ** -0.5)
    ws13 = rnd(2 * S, H, seed=4, dtype=torch.bfloat16, scale=H ** -0.5)
    ws2 = rnd(H, S, seed=5, dtype=torch.bfloat16, scale=S ** -0.5)
    nan = lambda *shape: torch.full(shape, float("nan"), dtype=torch.bfloat16, device=DEV)
    for tile_rows in (16, 32, 64):
        offsets, rows, dest, tile_map = dispatch(topk_e, E, tile_rows)
        act1, act2, sact = nan(T * k, mi), nan(T * k, mi), nan(T, S)
        ops.moe_grouped_mfma(x, w13, act1, offsets, rows, tile_map, tile_rows, True, 4)
        ops.moe_grouped_dual(x, w13, act2, offsets, rows, tile_map, tile_rows, x, ws13, sact, True)
        assert torch.equal(act1.view(torch.int16), act2.view(torch.int16))
        want = torch.nn.functional.silu(x.double() @ ws13[:S].double().T) * (x.double() @ ws13[S:].double().T)
        assert rel_err(sact, want) < 1.5e-2
        y1, y2, sout = nan(T * k, H), nan(T * k, H), nan(T, H)
        ops.moe_grouped_mfma(act1, w2, y1, offsets, None, tile_map, tile_rows, False, 4)
        ops.moe_grouped_dual(act2, w2, y2, offsets, None, tile_map, tile_rows, sact, ws2, sout, False)
        assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
        assert rel_err(sout, sact.double() @ ws2.double().T) < 1.5e-2
        assert rel_err(y2, grouped_reference(act2, w2, offsets.cpu(), None, False)) < 1.5e-2


@pytest.mark.parametrize("T,H,k,A", [(1, 64, 2, 2), (8, 2048, 4, 32), (21, 96, 3, 70), (5, 1000, 1, 5), (130, 72, 8, 1040)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_shared,gated", [(False, False), (True, False), (True, True)])
def test_expert_sum_add_and_norm_in_one_pass(T, H, k, A, dtype, with_shared, gated):
    """h += sum_s w[t, s] y[dest[t, s]] + gate[t] shared[t]; out = rmsnorm(h) * weight: against the two kernels one
    after the other (the sum rounded to the run's type in between, as they leave it) and against float64; with
    picked rows the stream is left alone."""
    from inferx_amd import ops
    g = torch.Generator().manual_seed(5)
    y = rnd(A, H, seed=1, dtype=dtype)
    dest = torch.stack([torch.randperm(A, generator=g)[:k] for _ in range(T)]).to(torch.int32).to(DEV)
    topk_w = torch.rand(T, k, generator=g).to(DEV)
    shared = rnd(T, H, seed=2, dtype=dtype) if with_shared else None
    gate = torch.rand(T, generator=g).to(DEV) if gated else None
    weight = (1.0 + rnd(H, seed=3, scale=0.2)).to(dtype)
    h0 = rnd(T, H, seed=4, scale=2.0)
    eps = 1e-5
    total = (topk_w.double()[:, :, None] * y.double()[dest.long()]).sum(1)
    if with_shared:
        total = total + (gate.double()[:, None] if gated else 1.0) * shared.double()
    h_want = h0.double() + total
    x_want = h_want * torch.rsqrt((h_want ** 2).mean(-1, keepdim=True) + eps) * weight.double()
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    h1, out1 = h0.clone(), torch.empty(T, H, dtype=dtype, device=DEV)
    ops.moe_combine_add_rmsnorm(h1, y, dest, topk_w, shared, gate, weight, out1, eps)
    assert rel_err(h1, h_want) < (1e-6 if dtype == torch.float32 else 4e-3) and rel_err(out1, x_want) < tol
    summed, h2, out2 = torch.empty(T, H, dtype=dtype, device=DEV), h0.clone(), torch.empty(T, H, dtype=dtype, device=DEV)
    ops.moe_combine(y, dest, topk_w, shared, gate, summed)
    ops.add_rmsnorm(h2, summed, weight, out2, eps)
    assert rel_err(h1, h2) < (1e-6 if dtype == torch.float32 else 4e-3) and rel_err(out1, out2) < tol
    rows = torch.tensor([T - 1, 0, T // 2, T // 2], dtype=torch.int32, device=DEV)
    h3, picked = h0.clone(), torch.empty(4, H, dtype=dtype, device=DEV)
    ops.moe_combine_add_rmsnorm(h3, y, dest, topk_w, shared, gate, weight, picked, eps, rows)
    assert torch.equal(h3, h0) and rel_err(picked, x_want[rows.long()]) < tol
