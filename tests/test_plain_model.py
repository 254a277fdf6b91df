"""What fixes the plain implementation beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine,
and invariants, each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_model as pm
import tiny

F64 = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, dtype=F64, generator=torch.Generator().manual_seed(seed))


def test_rms_norm_is_the_library_expression():
    x, w = rnd(5, 24), rnd(24, seed=1)
    want = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(pm.rms_norm(x, w, 1e-5), want, atol=1e-12)
    # eps sits inside the root, on the mean (not on the sum, not outside)
    tiny_x = torch.full((1, 4), 1e-4, dtype=F64)
    got = pm.rms_norm(tiny_x, torch.ones(4, dtype=F64), 1e-2)
    assert torch.allclose(got, tiny_x / math.sqrt(1e-8 + 1e-2), atol=1e-12)


def test_rope_is_a_complex_rotation_of_half_split_pairs():
    d, T = 16, 6
    x = rnd(T, 3, d)
    pos = torch.tensor([0, 1, 2, 5, 9, 100])
    got = pm.apply_rope(x, pos, 10000.0)
    # pair (j, j + d/2) as the complex number x_j + i x_{j+d/2}, times exp(i * pos * theta^(-2j/d))
    z = torch.complex(x[..., : d // 2], x[..., d // 2:])
    angle = pos[:, None].double() * pm.rope_frequencies(10000.0, d)[None, :]
    rot = z * torch.exp(1j * angle)[:, None, :]
    want = torch.cat([rot.real, rot.imag], dim=-1)
    assert torch.allclose(got, want, atol=1e-5)  # the angle is rounded to float32, as on the device
    assert torch.equal(got[0], x[0])  # position 0 is the identity
    assert torch.allclose(got.norm(dim=-1), x.norm(dim=-1), atol=1e-9)  # a rotation keeps lengths
    f = pm.rope_frequencies(10000.0, d)
    assert f[0] == 1.0 and abs(float(f[1]) - 10000.0 ** (-2.0 / d)) < 1e-7 and float(f[-1]) > 1e-4


def test_rope_fixed_vector_worked_by_hand():
    """d = 4, theta = 10000, position 1: frequencies 1 and 0.01; the row (1, 2, 3, 4) is the pairs (1, 3) at angle 1
    and (2, 4) at angle 0.01 (pairs (j, j + d/2), as the reference's own host twin pairs them,
    tests/kernel/mla_test.cc:239-263).  The numbers below were worked out by hand from cos 1 = 0.5403023058681398,
    sin 1 = 0.8414709848078965, cos 0.01 = 0.9999500004166653, sin 0.01 = 0.009999833334166664.  Interleaved pairs
    ((1, 2) at angle 1, (3, 4) at angle 0.01) give -1.1426..., a swapped sign gives +3.0647...: both fail."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]], dtype=F64)
    got = pm.apply_rope(x, torch.tensor([1]), 10000.0)[0, 0]
    want = torch.tensor([1 * 0.5403023058681398 - 3 * 0.8414709848078965,          # -1.98411064855...
                         2 * 0.9999500004166653 - 4 * 0.009999833334166664,        #  1.95990066749...
                         3 * 0.5403023058681398 + 1 * 0.8414709848078965,          #  2.46237790241...
                         4 * 0.9999500004166653 + 2 * 0.009999833334166664], dtype=F64)  # 4.01979966833...
    assert torch.allclose(want, torch.tensor([-1.98411064855555, 1.95990066749666, 2.46237790241231,
                                              4.01979966833500], dtype=F64), atol=1e-12)
    assert torch.allclose(got, want, atol=1e-6)  # frequency and angle are rounded to float32, as on the device
    interleaved = 1 * 0.5403023058681398 - 2 * 0.8414709848078965
    assert abs(float(got[0]) - interleaved) > 0.5


def test_rope_of_a_part_of_the_head_worked_by_hand():
    """Heads of 6, the trailing 4 rotated (the reference's own partial rotation takes the trailing part with the
    frequencies of the part's width, src/backends/cuda/ops/mla.cu:21-46): the row (9, 8, 1, 2, 3, 4) keeps 9 and 8
    and its tail is the vector of the test above.  Frequencies by the head's width (theta^(-2j/6)) would give the
    second pair the angle 0.0464 and 1.81 instead of 1.96; a rotation of the leading part would change the 9."""
    x = torch.tensor([[[9.0, 8.0, 1.0, 2.0, 3.0, 4.0]]], dtype=F64)
    got = pm.apply_rope_part(x, torch.tensor([1]), 10000.0, 2, 4)[0, 0]
    want = torch.tensor([9.0, 8.0, -1.98411064855555, 1.95990066749666, 2.46237790241231, 4.01979966833500], dtype=F64)
    assert torch.allclose(got, want, atol=1e-6)
    # the whole head as its part is the plain rotation; an empty stretch before or after changes nothing else
    y = rnd(5, 2, 8)
    pos = torch.tensor([0, 3, 4, 50, 7])
    assert torch.equal(pm.apply_rope_part(y, pos, 500.0, 0, 8), pm.apply_rope(y, pos, 500.0))
    part = pm.apply_rope_part(y, pos, 500.0, 2, 4)
    assert torch.equal(part[..., :2], y[..., :2]) and torch.equal(part[..., 6:], y[..., 6:])
    assert torch.equal(part[..., 2:6], pm.apply_rope(y[..., 2:6], pos, 500.0))


def test_attention_without_rotation_or_window_is_library_attention():
    T, heads, kv, d = 9, 6, 2, 8
    q, k, v = rnd(T, heads, d), rnd(T, kv, d, seed=1), rnd(T, kv, d, seed=2)
    got = pm.attention(q, k, v, torch.arange(T), 1 / math.sqrt(d))
    kk = k.repeat_interleave(heads // kv, dim=1)  # query head h reads kv head h // group
    vv = v.repeat_interleave(heads // kv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
    assert torch.allclose(got, want.transpose(0, 1), atol=1e-10)


def test_window():
    T, d = 12, 4
    q, k, v = rnd(T, 2, d), rnd(T, 1, d, seed=1), rnd(T, 1, d, seed=2)
    pos = torch.arange(T)
    full = pm.attention(q, k, v, pos, 0.5)
    assert torch.allclose(pm.attention(q, k, v, pos, 0.5, window=T), full)      # a window as long as the context
    assert torch.allclose(pm.attention(q, k, v, pos, 0.5, window=1), v.expand(T, 2, d))  # only the query's own key
    w3 = pm.attention(q, k, v, pos, 0.5, window=3)
    assert torch.allclose(w3[:3], full[:3]) and not torch.allclose(w3[3], full[3])  # W keys, the own one included
    # position p = 5 with W = 3 reads keys 3, 4, 5
    s = (k[3:6, 0] @ q[5, 0]) * 0.5
    assert torch.allclose(w3[5, 0], torch.softmax(s, 0) @ v[3:6, 0])


def test_gated_mlp_is_the_library_expression():
    x, g, u, dn = rnd(4, 10), rnd(14, 10, seed=1), rnd(14, 10, seed=2), rnd(10, 14, seed=3)
    assert torch.allclose(pm.gated_mlp(x, g, u, dn), F.linear(F.silu(F.linear(x, g)) * F.linear(x, u), dn), atol=1e-12)


def test_route_equal_logits_take_the_lowest_indices():
    # reference vector: tests/kernel/moe_test.cc:248-273 (E = 32, k = 2, all logits equal -> experts 0 and 1)
    x = torch.ones(3, 8, dtype=F64)
    wr = torch.full((32, 8), 0.25 / 8, dtype=F64)
    w, e = pm.route(x, wr, 2, renormalize=False)
    assert e.tolist() == [[0, 1]] * 3
    assert torch.allclose(w, torch.full((3, 2), 1 / 32, dtype=F64))


def test_route_weights():
    # reference: moe_test.cc:170-246 (renormalised sums to 1, un-normalised stays below)
    x, wr = rnd(7, 12), rnd(8, 12, seed=1)
    w, e = pm.route(x, wr, 3, renormalize=False)
    p = torch.softmax(x @ wr.T, -1)
    top = torch.topk(p, 3, dim=-1)
    assert torch.equal(e, top.indices) and torch.allclose(w, top.values)  # descending score
    assert (w.sum(-1) < 0.999).all()
    wn, en = pm.route(x, wr, 3, renormalize=True)
    assert torch.equal(en, e) and torch.allclose(wn.sum(-1), torch.ones(7, dtype=F64))
    assert torch.allclose(wn, w / w.sum(-1, keepdim=True))


def moe_weights(E, H, mi, si, seed=0):
    w = {"m.gate.weight": rnd(E, H, seed=seed)}
    for e in range(E):
        w[f"m.experts.{e}.gate_proj.weight"] = rnd(mi, H, seed=seed + 10 + e)
        w[f"m.experts.{e}.up_proj.weight"] = rnd(mi, H, seed=seed + 50 + e)
        w[f"m.experts.{e}.down_proj.weight"] = rnd(H, mi, seed=seed + 90 + e)
    if si:
        w["m.shared_expert.gate_proj.weight"] = rnd(si, H, seed=seed + 1)
        w["m.shared_expert.up_proj.weight"] = rnd(si, H, seed=seed + 2)
        w["m.shared_expert.down_proj.weight"] = rnd(H, si, seed=seed + 3)
        w["m.shared_expert_gate.weight"] = rnd(1, H, seed=seed + 4)
    return w


def expert(w, e, x):
    p = f"m.experts.{e}."
    return pm.gated_mlp(x, w[p + "gate_proj.weight"], w[p + "up_proj.weight"], w[p + "down_proj.weight"])


def test_moe_special_cases():
    E, H, mi = 4, 6, 5
    x = rnd(5, H, seed=7) * 0.3
    w = moe_weights(E, H, mi, 0)
    # k = E with renormalisation: the softmax-weighted sum of ALL experts
    p = torch.softmax(x @ w["m.gate.weight"].T, -1)
    want = sum(p[:, e:e + 1] * expert(w, e, x) for e in range(E))
    assert torch.allclose(pm.moe_block(x, w, "m.", E, E, True, 0), want, atol=1e-10)
    # one expert: the plain MLP with weight 1
    w1 = moe_weights(1, H, mi, 0)
    assert torch.allclose(pm.moe_block(x, w1, "m.", 1, 1, False, 0), expert(w1, 0, x), atol=1e-12)
    # identical experts and renormalisation: the single MLP, whatever is chosen
    same = dict(w)
    for e in range(1, E):
        for n in ("gate_proj", "up_proj", "down_proj"):
            same[f"m.experts.{e}.{n}.weight"] = same[f"m.experts.0.{n}.weight"]
    assert torch.allclose(pm.moe_block(x, same, "m.", E, 2, True, 0), expert(same, 0, x), atol=1e-10)
    # without renormalisation the sum is scaled by the chosen probabilities' sum (< 1)
    ws, _ = pm.route(x, same["m.gate.weight"], 2, False)
    assert torch.allclose(pm.moe_block(x, same, "m.", E, 2, False, 0), ws.sum(-1, keepdim=True) * expert(same, 0, x),
                          atol=1e-10)


def test_shared_expert_gate():
    E, H, mi, si = 3, 6, 4, 7
    x = rnd(4, H, seed=3) * 0.3
    w = moe_weights(E, H, mi, si)
    routed = pm.moe_block(x, {k: v for k, v in w.items() if "shared" not in k}, "m.", E, 2, False, 0)
    shared = pm.gated_mlp(x, w["m.shared_expert.gate_proj.weight"], w["m.shared_expert.up_proj.weight"],
                          w["m.shared_expert.down_proj.weight"])
    # a zero gate weight gives sigmoid(0) = 0.5
    w0 = dict(w)
    w0["m.shared_expert_gate.weight"] = torch.zeros(1, H, dtype=F64)
    assert torch.allclose(pm.moe_block(x, w0, "m.", E, 2, False, si), routed + 0.5 * shared, atol=1e-12)
    g = torch.sigmoid(x @ w["m.shared_expert_gate.weight"].T)
    got = pm.moe_block(x, w, "m.", E, 2, False, si)
    assert torch.allclose(got, routed + g * shared, atol=1e-12)
    assert ((got - routed).abs().sum(-1) > 0).all()  # the shared expert changes every row (moe_test.cc:607-702)


def test_greedy_and_support():
    # reference vectors: tests/unit/host_sampling_test.cc:12-17 ({1,4,2} -> 1), :34-53 (top-k 2 -> {0, 1})
    assert pm.greedy(torch.tensor([1.0, 4.0, 2.0])) == 1
    assert pm.greedy(torch.tensor([3.0, 3.0, 1.0])) == 0  # lowest index on ties
    row = torch.tensor([5.0, 4.0, 1.0, 0.0])
    assert pm.sampling_support(row, 0.8, top_k=2) == [0, 1]
    assert pm.sampling_support(row, 1.0, min_p=0.3) == [0, 1]      # p1/p0 = e^-1 = 0.37 stays, p2/p0 = e^-4 goes
    assert pm.sampling_support(row, 1.0, top_p=0.5) == [0]         # p0 = 0.72 alone reaches 0.5
    assert pm.sampling_support(row, 1.0, top_p=0.9) == [0, 1]
    assert pm.sampling_support(row, 1.0) == [0, 1, 2, 3]


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = tmp_path_factory.mktemp("plain_b")
    tiny.make_folder(tiny.CONFIG_B, 3, str(d), "float32")
    return tiny.read_folder(str(d))


def test_which_layer_is_which():
    assert [pm.is_moe_layer(tiny.CONFIG_B, l) for l in range(4)] == [False, True, False, True]
    assert [pm.window_of_layer(tiny.CONFIG_B, l) for l in range(4)] == [0, 0, 16, 16]
    assert all(pm.is_moe_layer(tiny.CONFIG_A, l) for l in range(2))


def test_only_distances_count(model_b):
    # a shift of all positions changes nothing: fails if q and k turn in different senses or are paired differently
    cfg, w = model_b
    toks = tiny.random_tokens(30, cfg["vocab_size"], 4)
    base = pm.forward(cfg, w, toks)
    shifted = pm.forward(cfg, w, toks, positions=range(37, 67))
    assert float((base - shifted).abs().max()) < 2e-4 * float(base.abs().max())  # float32 angles at larger positions


def test_causal_and_windowed(model_b):
    cfg, w = model_b
    toks = tiny.random_tokens(30, cfg["vocab_size"], 5)
    base = pm.forward(cfg, w, toks)
    other = list(toks)
    other[25] = (other[25] + 1) % cfg["vocab_size"]
    changed = pm.forward(cfg, w, other)
    assert torch.equal(base[:25], changed[:25]) and not torch.allclose(base[25], changed[25])
    # without the window the result differs once the context exceeds it
    no_window = dict(cfg, use_sliding_window=False)
    full = pm.forward(no_window, w, toks)
    assert torch.allclose(full[:16], base[:16], atol=1e-12) and not torch.allclose(full[20:], base[20:], atol=1e-6)


def test_norms_and_residuals_sit_where_the_reference_puts_them(model_b):
    # with every output projection zero, nothing is added to the stream: logits = head(norm(embed))
    cfg, w = model_b
    z = {k: (torch.zeros_like(v) if k.endswith(("o_proj.weight", "down_proj.weight")) else v) for k, v in w.items()}
    toks = tiny.random_tokens(6, cfg["vocab_size"], 6)
    emb = z["model.embed_tokens.weight"].double()[torch.tensor(toks)]
    want = pm.rms_norm(emb, z["model.norm.weight"].double(), cfg["rms_norm_eps"]) @ z["model.embed_tokens.weight"].double().T
    assert torch.allclose(pm.forward(cfg, z, toks), want, atol=1e-12)
    # one layer, by hand: h1 = e + attn(norm(e)); out = h1 + ffn(norm(h1)) -- pre-norm, residual from the un-normed stream
    one = dict(cfg, num_hidden_layers=1, mlp_only_layers=[0], use_sliding_window=False)
    e = w["model.embed_tokens.weight"].double()[torch.tensor(toks[:1])]
    p = "model.layers.0."
    x = pm.rms_norm(e, w[p + "input_layernorm.weight"].double(), cfg["rms_norm_eps"])
    v = x @ w[p + "self_attn.v_proj.weight"].double().T + w[p + "self_attn.v_proj.bias"].double()
    att = v.view(1, 1, 32).expand(1, 3, 32).reshape(1, 96)  # one token: softmax over itself; 3 heads share the kv head
    h1 = e + att @ w[p + "self_attn.o_proj.weight"].double().T
    x2 = pm.rms_norm(h1, w[p + "post_attention_layernorm.weight"].double(), cfg["rms_norm_eps"])
    h2 = h1 + pm.gated_mlp(x2, w[p + "mlp.gate_proj.weight"].double(), w[p + "mlp.up_proj.weight"].double(),
                           w[p + "mlp.down_proj.weight"].double())
    want = pm.rms_norm(h2, w["model.norm.weight"].double(), cfg["rms_norm_eps"]) @ w["model.embed_tokens.weight"].double().T
    assert torch.allclose(pm.forward(one, w, toks[:1]), want, atol=1e-12)


def test_bfloat16_storage_mode(model_b):
    """The plain implementation with every stored activation rounded to bfloat16: the same model up to rounding
    (a few parts in a thousand of the largest logit), not bit-equal, and untouched when nothing is rounded."""
    cfg, w = model_b
    toks = tiny.random_tokens(24, cfg["vocab_size"], 9)
    base = pm.forward(cfg, w, toks)
    assert torch.equal(pm.forward(cfg, w, toks, rnd=pm.no_rounding), base)
    scores = []
    stored = pm.forward(cfg, w, toks, rnd=pm.to_bfloat16_and_back, router_scores=scores)
    moved = float((stored - base).abs().max()) / float(base.abs().max())
    assert 1e-5 < moved < 3e-2
    assert len(scores) == 2 and scores[0].shape == (24, cfg["num_experts"])  # config B has two sparse layers
    assert torch.equal(scores[0], pm.to_bfloat16_and_back(scores[0]))       # the scores are stored rounded too
