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
TIE_SPREADS = 4  # how many spreads of a score difference under bfloat16 count as a near tie


def case(name):
    """(config dict, weights on the device, float64 weights, prompts, expected logits, the plain selection, the
    near-tie bound per layer, bfloat16 tolerance), made once per shape.

    The bfloat16 tolerance is derived, not chosen: the plain implementation is run a second time with every stored
    activation rounded to bfloat16 (the reference's bfloat16 model) and the experts of the first run; how far that
    moves the logits is the error that bfloat16 alone brings, and an engine that also computes in bfloat16, in
    another order, may differ from the float64 result by twice that (the reference's way:
    scripts/gen_reference_logits.py:51-55).  The same second run says how much a router score moves under bfloat16
    (a robust spread per layer): two experts whose float64 scores differ by less than four such spreads of a
    difference are a near tie, where a bfloat16 run may choose either (the reference says the same of its own
    models, tests/kernel/deepseek_v2_reference_test.cc:24-28)."""
    if name not in _cases:
        from inferx_amd.config import config_from_dict
        from inferx_amd.parts import build_model
        from inferx_amd.weights import random_tensors
        _cases.clear()  # one shape's float64 weights at a time
        raw = SHAPES[name]
        model = build_model(config_from_dict(raw).model_spec())
        weights = random_tensors(model, 5, "bfloat16", device="cuda:0")
        wide = pm.Widened({name_: t.cpu() for name_, t in weights.items()})
        prompts = {f"r{i}": tiny.random_tokens(n, raw["vocab_size"], seed=300 + i) for i, n in enumerate(PROMPT_LENGTHS)}
        expected, chosen, moved = {}, {}, None
        gap = 0.0
        for rid, toks in prompts.items():
            z64, z16, chosen[rid] = [], [], []
            expected[rid] = pm.forward(raw, wide, toks, router_scores=z64, experts_out=chosen[rid])
            stored = pm.forward(raw, wide, toks, rnd=pm.to_bfloat16_and_back, router_scores=z16, experts=chosen[rid])
            gap = max(gap, float((stored - expected[rid]).abs().max()))
            diffs = [(a - b).abs().flatten() for a, b in zip(z16, z64)]
            moved = diffs if moved is None else [torch.cat([m, d]) for m, d in zip(moved, diffs)]
        gap /= max(float(e.abs().max()) for e in expected.values())
        # per layer: the spread of one score under bfloat16; a difference of two scores has sqrt(2) of it
        bounds = [TIE_SPREADS * 2 ** 0.5 * 1.4826 * float(m.median()) for m in moved]
        print(f"{name}: bfloat16 storage alone moves the logits by {gap:.2e} of the largest, so the bfloat16 "
              f"tolerance is {2 * gap:.2e}; near ties: scores closer than {', '.join(f'{b:.2e}' for b in bounds)}",
              flush=True)
        _cases[name] = (raw, weights, wide, prompts, expected, chosen, bounds, 2 * gap)
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


class ChosenExperts:
    """What the engine's router chose, per (request, position) and sparse layer: every step's batch is noted when it
    is run, and every routing call of that step (they come in layer order) has its selection read back."""

    def __init__(self, runner, monkeypatch):
        from inferx_amd.parts.moe import MoeFeedForward
        self.by_place = {}
        self._rows, self._calls = None, 0
        real_step, real_route = runner.step, MoeFeedForward.route_and_dispatch
        owner = self

        def step(batch):
            owner._rows = [(batch.request_ids[int(s)], int(p)) for s, p in zip(batch.seq_of_token, batch.positions)]
            owner._calls = 0
            return real_step(batch)

        def route_and_dispatch(part, ctx, x, tile_rows, norm=None, always=0):
            out = real_route(part, ctx, x, tile_rows, norm, always)
            if torch.cuda.is_current_stream_capturing():
                return out
            layer, owner._calls = owner._calls, owner._calls + 1
            # (the chosen experts: further columns hold the shared expert's pieces in steps that take them along)
            for place, experts in zip(owner._rows, out[1][:, :part.top_k].cpu().tolist()):
                owner.by_place.setdefault(place, {})[layer] = experts
            return out
        runner.step = step
        monkeypatch.setattr(MoeFeedForward, "route_and_dispatch", route_and_dispatch)

    def of_request(self, rid, length, layers):
        """[layers] tensors [length, k]."""
        return [torch.tensor([self.by_place[(rid, pos)][l] for pos in range(length)]) for l in range(layers)]


def expected_with_the_engines_experts(name, chosen_by_engine, what):
    """The plain logits per request, with the engine's selection wherever it differs from the plain one; a selection
    that differs by more than a near tie (in the scores of the plain run that has the engine's selections in the
    layers before) fails.  Returns (expected, places that differed)."""
    raw, _, wide, prompts, expected, chosen, bounds, _ = case(name)
    out, differed = {}, 0
    for rid, toks in prompts.items():
        engine = chosen_by_engine.of_request(rid, len(toks), len(bounds))
        same = [bool((e.sort(-1).values == c.sort(-1).values).all()) for e, c in zip(engine, chosen[rid])]
        if all(same):
            out[rid] = expected[rid]
            continue
        scores = []
        out[rid] = pm.forward(raw, wide, toks, router_scores=scores, experts=engine)
        for l, (z, e) in enumerate(zip(scores, engine)):
            k = e.shape[1]
            plain = torch.topk(z, k, dim=-1).indices
            for pos in range(len(toks)):
                theirs, ours = set(e[pos].tolist()), set(plain[pos].tolist())
                if theirs == ours:
                    continue
                differed += 1
                lost = max(float(z[pos, i]) for i in ours - theirs)    # the best that the engine left out ...
                taken = min(float(z[pos, i]) for i in theirs - ours)   # ... and the worst that it took instead
                assert lost - taken < bounds[l], \
                    (f"{what}: request {rid} position {pos} layer {l}: the engine chose experts {sorted(theirs - ours)} "
                     f"over {sorted(ours - theirs)}, whose scores are apart by {lost - taken:.3e}: no near tie "
                     f"(bound {bounds[l]:.3e})")
    return out, differed


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SHAPES))  # (the slower-changing parameter: a shape's case is made once)
def test_real_layer_sizes_four_ways(name, dtype, monkeypatch):
    """Every place is compared in both types.  Where the bfloat16 engine chose other experts than the plain
    implementation, the choice must be a near tie, and the place is then compared with the plain implementation run
    with the engine's choice; no place is left out."""
    raw, _, _, prompts, expected, _, _, bf16_tol = case(name)
    tol = ru.FP32_TOL if dtype == "float32" else bf16_tol
    runner = make_runner(name, dtype)
    if dtype == "bfloat16":
        # the selections are read back call by call, so no step is replayed from a graph at first (below they are);
        # steps of one token per request are planned as their recorded form is
        runner.capture_after = 10 ** 9
        chosen = ChosenExperts(runner, monkeypatch)
    ways = [("whole", ru.whole(prompts)), ("last 32 one by one", ru.tail_decoded(prompts, 32)),
            ("portions", ru.chunked(prompts)), ("mixed", ru.mixed(prompts, seed=8, max_tokens=MAX_TOKENS))]
    for how, steps in ways:
        owners = {}
        differed = 0
        if dtype == "bfloat16":
            chosen.by_place.clear()
        got = ru.replay(runner, steps, page_owners=owners)
        want = expected
        if dtype == "bfloat16":
            want, differed = expected_with_the_engines_experts(name, chosen, f"{name} {how}")
        worst = ru.compare(got, want, tol, f"{name} {dtype} {how}")
        print(f"{name} {dtype} {how}: worst {worst:.2e} of the largest logit over all {len(got)} places"
              + (f"; {differed} selections fell the other way at a near tie" if dtype == "bfloat16" else ""), flush=True)
        assert all(p.used_pages == 0 for p in runner.cache.pools)
        if how == "mixed":
            assert any(len(rids) > 1 for rids in owners.values()), "no page was used again"
        if dtype == "bfloat16" and how == "last 32 one by one":
            # the same steps with their one-token steps replayed from graphs: the same bits
            runner.capture_after = 2
            again = ru.replay(runner, steps)
            runner.capture_after = 10 ** 9
            assert runner._graphs, "no step was replayed from a graph"
            runner._graphs.clear()
            assert all(torch.equal(again[place], row) for place, row in got.items()), \
                f"{name}: a step replayed from a graph gives other bits than the same step run kernel by kernel"
