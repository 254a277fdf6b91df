"""The whole model at the layer sizes of real checkpoints against the plain implementation: one and two layers of
the Qwen1.5-MoE-A2.7B shape (width 2048, 16 heads, 60 experts of 1408, 4 per token, shared expert of 5632) and one
layer of the Qwen2-57B-A14B shape (width 3584, 28 query heads on 4 key/value heads, 64 experts of 2560, 8 per token,
shared expert of 20480), both with the full vocabulary of 151,936, in float32 and in bfloat16, each request whole,
with its last 32 tokens one by one, in portions, and mixed with so few pages that they are used again.  The tiny
configurations never reach the kernels' paths for these sizes (wide expert tiles, grouped query heads of seven,
the shared expert beside the routed ones, the streaming head product).

Weights are drawn on the device in bfloat16 and handed to the runner directly (a float32 run widens them, which is
exact), so both runs and the plain implementation see the same numbers and no folder of gigabytes is written.
(The reference tests its own whole models the same way: tests/kernel/deepseek_v2_model_test.cc:615-770.)"""
import pytest
import torch

import plain_model as pm
import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu

A27B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "num_hidden_layers": 2, "hidden_size": 2048,
    "num_attention_heads": 16, "num_key_value_heads": 16, "num_experts": 60, "num_experts_per_tok": 4,
    "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632, "intermediate_size": 5632,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False, "vocab_size": 151936,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 4096, "use_sliding_window": False,
    "tie_word_embeddings": False,
}
B57 = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "num_hidden_layers": 1, "hidden_size": 3584,
    "num_attention_heads": 28, "num_key_value_heads": 4, "num_experts": 64, "num_experts_per_tok": 8,
    "moe_intermediate_size": 2560, "shared_expert_intermediate_size": 20480, "intermediate_size": 18944,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False, "vocab_size": 151936,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 8192, "use_sliding_window": False,
    "tie_word_embeddings": False,
}
SHAPES = {"a27b_1_layer": dict(A27B, num_hidden_layers=1), "a27b_2_layers": A27B, "57b_1_layer": B57,
          "57b_2_layers": dict(B57, num_hidden_layers=2)}
PROMPT_LENGTHS = (40, 150, 300)
MAX_TOKENS = 384  # the pool: the longest request alone, or the two others together


_cases = {}


def case(name):
    """(config dict, weights on the device, prompts, expected logits, near ties, bfloat16 tolerance), made once per
    shape.

    The bfloat16 tolerance is derived, not chosen: the plain implementation is run a second time with every stored
    activation rounded to bfloat16 (the reference's bfloat16 model); how far that moves the logits is the error
    that bfloat16 alone brings, and an engine that also computes in bfloat16, in another order, may differ from the
    float64 result by twice that (the reference's way: scripts/gen_reference_logits.py:51-55).  The same second
    run says how much a router score moves under bfloat16 (a robust spread per layer); where the last chosen
    expert leads the first one left out by less than four such spreads of a difference, bfloat16 may choose the
    other expert, which moves that token's logits by far more than rounding, so those places are left out of the
    bfloat16 comparison (never of the float32 one).  With 8 experts of 64 per token and two layers that is most
    places; what is left is still a hundred rows of the full vocabulary per way of running."""
    if name not in _cases:
        from inferx_amd.config import config_from_dict
        from inferx_amd.parts import build_model
        from inferx_amd.weights import random_tensors
        _cases.clear()  # one shape's float64 weights at a time
        raw = SHAPES[name]
        k = raw["num_experts_per_tok"]
        model = build_model(config_from_dict(raw).model_spec())
        weights = random_tensors(model, 5, "bfloat16", device="cuda:0")
        wide = pm.Widened({name_: t.cpu() for name_, t in weights.items()})
        prompts = {f"r{i}": tiny.random_tokens(n, raw["vocab_size"], seed=300 + i) for i, n in enumerate(PROMPT_LENGTHS)}
        expected, stored, z64, z16 = {}, {}, {}, {}
        for rid, toks in prompts.items():
            z64[rid], z16[rid] = [], []
            expected[rid] = pm.forward(raw, wide, toks, router_scores=z64[rid])
            stored[rid] = pm.forward(raw, wide, toks, rnd=pm.to_bfloat16_and_back, router_scores=z16[rid])
        layers = len(next(iter(z64.values())))
        ties = set()
        for l in range(layers):
            # (measured where no earlier layer was a near tie: there the rounded run may already have gone another way)
            clear = {rid: torch.tensor([(rid, p) not in ties for p in range(len(prompts[rid]))]) for rid in prompts}
            moved = torch.cat([(z16[rid][l] - z64[rid][l])[clear[rid]].abs().flatten() for rid in prompts])
            spread = 1.4826 * float(moved.median())  # of one score; a difference of two has sqrt(2) of it
            for rid in prompts:
                top = torch.topk(z64[rid][l], k + 1, dim=-1).values
                lead = top[:, k - 1] - top[:, k]
                ties |= {(rid, int(p)) for p in torch.nonzero(lead < 4 * 2 ** 0.5 * spread).flatten()}
        total = sum(PROMPT_LENGTHS)
        assert len(ties) < 0.8 * total, "too many near ties for the comparison to mean much"
        scale = max(float(e.abs().max()) for e in expected.values())
        gap = max(float((stored[rid][pos] - expected[rid][pos]).abs().max()) / scale
                  for rid in prompts for pos in range(len(prompts[rid])) if (rid, pos) not in ties)
        print(f"{name}: {len(ties)} near ties of {total} places; bfloat16 storage alone moves the logits by {gap:.2e} "
              f"of the largest, so the bfloat16 tolerance is {2 * gap:.2e}", flush=True)
        _cases[name] = (raw, weights, prompts, expected, ties, 2 * gap)
    return _cases[name]


def make_runner(name, dtype):
    """A runner on the shape's weights: bfloat16 as drawn, or widened to float32 (exact)."""
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    raw, weights = case(name)[:2]
    rt = Runtime(dtype)
    placed = {k: rt.place(v) for k, v in weights.items()}
    return ModelRunner(config_from_dict(raw), placed, rt, page_size=16, num_pages=MAX_TOKENS // 16, max_requests=4,
                       max_seq_len=MAX_TOKENS)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))  # (the slower-changing parameter: a shape's case is made once)
def test_real_layer_sizes_four_ways(name, dtype):
    raw, _, prompts, expected, ties, bf16_tol = case(name)
    tol = ru.FP32_TOL if dtype == "float32" else bf16_tol
    skip = ties if dtype == "bfloat16" else set()
    runner = make_runner(name, dtype)
    ways = [("whole", ru.whole(prompts)), ("last 32 one by one", ru.tail_decoded(prompts, 32)),
            ("portions", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=8, max_tokens=MAX_TOKENS))]
    for how, steps in ways:
        owners = {}
        got = ru.replay(runner, steps, page_owners=owners)
        worst = ru.compare(got, expected, tol, f"{name} {dtype} {how}", skip)
        print(f"{name} {dtype} {how}: worst {worst:.2e} of the largest logit", flush=True)
        assert all(p.used_pages == 0 for p in runner.cache.pools)
        if how == "mixed":
            assert any(len(rids) > 1 for rids in owners.values()), "no page was used again"
