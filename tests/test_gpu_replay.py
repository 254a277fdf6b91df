"""The engine against the plain implementation, four ways of running each request,
in float32 and in bfloat16, on two tiny configurations that differ in every size."""
import pytest
import torch

import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu

PROMPT_LENGTHS = {"A": (5, 9, 17, 70), "B": (7, 23, 40, 75), "C": (11, 50, 29, 70), "D": (3, 37, 66)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in tiny.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            d = tmp_path_factory.mktemp(f"model_{name}_{dtype}")
            tiny.make_folder(cfg, seed=11, out_dir=str(d), dtype=dtype)
            out[(name, dtype)] = str(d)
    return out


def prompts_for(name):
    cfg = tiny.CONFIGS[name]
    return {f"r{i}": tiny.random_tokens(n, cfg["vocab_size"], seed=100 + i)
            for i, n in enumerate(PROMPT_LENGTHS[name])}


_expected_cache = {}


def expected_for(folders, name, dtype):
    key = (name, dtype)
    if key not in _expected_cache:
        cfg, weights = tiny.read_folder(folders[key])
        _expected_cache[key] = ru.expected_logits(cfg, weights, prompts_for(name))
    return _expected_cache[key]


_ties_cache = {}


def ties_for(folders, name, dtype):
    """Near ties of the routing: left out of bfloat16 comparisons only."""
    if dtype == "float32":
        return set()
    if name not in _ties_cache:
        cfg, weights = tiny.read_folder(folders[(name, dtype)])
        _ties_cache[name] = ru.near_ties(cfg, weights, prompts_for(name))
        total = sum(len(p) for p in prompts_for(name).values())
        assert len(_ties_cache[name]) < 0.15 * total, "too many near ties for the comparison to mean much"
    return _ties_cache[name]


def make_runner(folders, name, dtype, num_pages=64, page_size=16):
    from inferx_amd.engine.runner import ModelRunner
    return ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=page_size, num_pages=num_pages,
                                      max_requests=4, max_seq_len=num_pages * page_size)


def tol_of(dtype):
    return ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole(folders, name, dtype):
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, ru.whole(prompts_for(name)))
    worst = ru.compare(got, expected_for(folders, name, dtype), tol_of(dtype), f"whole {name} {dtype}",
                       ties_for(folders, name, dtype))
    print(f"whole {name} {dtype}: worst {worst:.2e}")


@pytest.mark.parametrize("name", ["A", "B"])
def test_bfloat16_run_keeps_tensors_stored_in_32_bits(folders, name):
    """A folder stored in float32, run with dtype bfloat16: every tensor stays float32 (activations are
    bfloat16), so the result is closer to the plain implementation on the float32 weights than bfloat16 weights
    would allow; and it goes through the kernels' mixed-type paths."""
    from inferx_amd.engine.runner import ModelRunner
    runner = ModelRunner.from_directory(folders[(name, "float32")], dtype="bfloat16", page_size=16, num_pages=64,
                                        max_requests=4, max_seq_len=1024)
    assert runner.model.embedding.weight.dtype == torch.float32
    assert runner.model.blocks[-1].mixer.w_qkv.dtype == torch.float32
    prompts = prompts_for(name)
    for steps in (ru.whole(prompts), ru.tail_decoded(prompts, 8), ru.mixed(prompts, seed=3)):
        got = ru.replay(runner, steps)
        ru.compare(got, expected_for(folders, name, "float32"), ru.BF16_TOL, f"mixed types {name}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_last_tokens_one_by_one(folders, name, dtype):
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, ru.tail_decoded(prompts_for(name), 32))
    ru.compare(got, expected_for(folders, name, dtype), tol_of(dtype), f"tail {name} {dtype}",
               ties_for(folders, name, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_portions_of_changing_size(folders, name, dtype):
    runner = make_runner(folders, name, dtype)
    got = ru.replay(runner, ru.chunked(prompts_for(name)))
    ru.compare(got, expected_for(folders, name, dtype), tol_of(dtype), f"chunked {name} {dtype}",
               ties_for(folders, name, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_mixed_with_few_pages(folders, name, dtype):
    prompts = prompts_for(name)
    # room for about two of the longer requests: pages are given back and used again
    max_tokens = 192
    runner = make_runner(folders, name, dtype, num_pages=max_tokens // 16)
    owners = {}
    steps = ru.mixed(prompts, seed=8, max_tokens=max_tokens)
    assert any(len(s["entries"]) > 1 and {len(e[1]) for e in s["entries"]} & {1} and
               max(len(e[1]) for e in s["entries"]) > 1 for s in steps), "no step mixes a portion with a single token"
    got = ru.replay(runner, steps, page_owners=owners)
    reused = [key for key, rids in owners.items() if len(rids) > 1]
    assert reused, "no physical page served two requests: the pool is too large for this test to bite"
    ru.compare(got, expected_for(folders, name, dtype), tol_of(dtype), f"mixed {name} {dtype}",
               ties_for(folders, name, dtype))
    assert all(p.used_pages == 0 for p in runner.cache.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
@pytest.mark.parametrize("min_workgroups", [0, None, "slices"])
def test_decoding_requests_beside_long_portions(folders, name, dtype, min_workgroups, monkeypatch):
    """Steps of more than 128 tokens in prompt portions with requests beside them that bring one to three tokens,
    before, between and after the portions' rows: in bfloat16 the portions' queries and the others' go to
    different attention kernels within one step (min_workgroups 0: also with as few query tiles as a tiny model
    has; None: the rule as it is, which sends such steps to one kernel; "slices": the portions' keys are cut into
    slices of one round, as those of long contexts are)."""
    from inferx_amd.parts import attention
    if min_workgroups == "slices":
        monkeypatch.setattr(attention, "PREFILL_SLICED_MIN_ROUNDS", 2)
        monkeypatch.setattr(attention, "PREFILL_SLICE_ROUNDS", 1)
    elif min_workgroups is not None:
        monkeypatch.setattr(attention, "PREFILL_MIN_WORKGROUPS", min_workgroups)
    cfg = tiny.CONFIGS[name]
    lengths = {"r0": 200, "r1": 60, "r2": 236}
    prompts = {rid: tiny.random_tokens(n, cfg["vocab_size"], seed=300 + i) for i, (rid, n) in enumerate(lengths.items())}
    at = {rid: 0 for rid in prompts}
    plan = [[("r1", 40), ("r2", 30)],
            [("r1", 1), ("r0", 150), ("r2", 3)],
            [("r0", 48), ("r1", 1), ("r2", 100)],
            [("r2", 1), ("r1", 2), ("r0", 2)],
            [("r1", 16), ("r2", 102)]]
    steps = []
    for entries in plan:
        step = {"entries": [], "end": []}
        for rid, n in entries:
            step["entries"].append((rid, prompts[rid][at[rid]:at[rid] + n], list(range(n))))
            at[rid] += n
            if at[rid] == lengths[rid]:
                step["end"].append(rid)
        steps.append(step)
    assert at == lengths
    raw, weights = tiny.read_folder(folders[(name, dtype)])
    want = ru.expected_logits(raw, weights, prompts)
    skip = ru.near_ties(raw, weights, prompts) if dtype == "bfloat16" else set()
    runner = make_runner(folders, name, dtype, num_pages=40)
    ru.compare(ru.replay(runner, steps), want, tol_of(dtype), f"beside portions {name} {dtype}", skip)
    assert all(p.used_pages == 0 for p in runner.cache.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [1, 2, 3, 5, 8, 13, 19, 34])
def test_random_configurations(tmp_path, seed, dtype, monkeypatch):
    """Configurations drawn at random from what the architecture allows (head sizes up to 256 and some that are no
    multiple of 16, odd widths, up to 130 experts, pages of 16 to 64, windows): portions of changing size and
    mixed steps against the plain implementation.  (Odd seeds: prompt portions go to the attention kernel for
    many query tiles also with the few tiles that a tiny model has.)"""
    from inferx_amd.engine.runner import ModelRunner
    if seed % 2:
        from inferx_amd.parts import attention
        monkeypatch.setattr(attention, "PREFILL_MIN_WORKGROUPS", 0)
    cfg = tiny.random_config(seed)
    page = cfg.pop("_page_size")
    tiny.make_folder(cfg, seed=seed, out_dir=str(tmp_path), dtype=dtype)
    raw, weights = tiny.read_folder(str(tmp_path))
    prompts = {f"r{i}": tiny.random_tokens(n, cfg["vocab_size"], seed=7 * seed + i) for i, n in enumerate((5, 37, 70, 150))}
    want = ru.expected_logits(raw, weights, prompts)
    skip = ru.near_ties(raw, weights, prompts) if dtype == "bfloat16" else set()
    for how, steps in (("whole", ru.whole(prompts)), ("portions", ru.chunked(prompts)),
                       ("mixed", ru.mixed(prompts, seed=seed, max_live=4))):
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=page, num_pages=4 * (160 // page + 2),
                                            max_requests=4, max_seq_len=256)
        ru.compare(ru.replay(runner, steps), want, (ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL), f"seed {seed} {dtype} {how}", skip=skip)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,requests", [("A", 40), ("B", 64), ("D", 33)])
def test_many_requests_decoding_together(folders, name, dtype, requests):
    """More decoding requests in a step than the few-rows kernels take (so the dense products go to the vendor's
    library, also inside the captured graph of the step): prompts of a few tokens, then six tokens each, one a step."""
    from inferx_amd.engine.runner import ModelRunner
    cfg = tiny.CONFIGS[name]
    raw, weights = tiny.read_folder(folders[(name, dtype)])
    prompts = {f"r{i}": tiny.random_tokens(4 + i % 5 + 6, cfg["vocab_size"], seed=300 + i) for i in range(requests)}
    want = ru.expected_logits(raw, weights, prompts)
    skip = ru.near_ties(raw, weights, prompts) if dtype == "bfloat16" else set()
    steps = [{"entries": [(rid, toks[:-6], list(range(len(toks) - 6)))], "end": []} for rid, toks in prompts.items()]
    for i in range(6):
        steps.append({"entries": [(rid, toks[len(toks) - 6 + i:len(toks) - 5 + i], [0]) for rid, toks in prompts.items()],
                      "end": list(prompts) if i == 5 else []})
    runner = ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=16, num_pages=2 * requests,
                                        max_requests=requests, max_seq_len=64)
    ru.compare(ru.replay(runner, steps), want, tol_of(dtype), f"{requests} requests {name} {dtype}", skip)
    assert runner._graphs, "the steps of one token per request were not replayed from a graph"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_shapes_come_and_go(folders, dtype):
    """A shape of one-token steps is captured when it comes for the third time and runs kernel by kernel before;
    the runner keeps a bounded number of graphs, the least recently replayed goes first; the graphs leave their
    logits in one buffer.  Four requests that end one after the other pass through the shapes 4, 3, 2, 1 and, with
    new requests, come back to 2: every logit as expected whichever way its step ran."""
    from inferx_amd.engine.runner import ModelRunner
    name = "A"
    cfg = tiny.CONFIGS[name]
    raw, weights = tiny.read_folder(folders[(name, dtype)])
    lens = {"a": 39, "b": 43, "c": 47, "d": 51, "e": 49, "f": 49}  # (contexts of 35 to 51: one bucket of contexts)
    prompts = {rid: tiny.random_tokens(n, cfg["vocab_size"], seed=500 + i) for i, (rid, n) in enumerate(lens.items())}
    want = ru.expected_logits(raw, weights, prompts)
    skip = ru.near_ties(raw, weights, prompts) if dtype == "bfloat16" else set()
    first = ["a", "b", "c", "d"]
    steps = [{"entries": [(rid, prompts[rid][:34], list(range(34)))], "end": []} for rid in first]
    at = {rid: 34 for rid in first}
    live = list(first)
    while live:  # one token each; the shortest ends first: 5 steps of four requests, then 4 of three, of two, of one
        entries = [(rid, prompts[rid][at[rid]:at[rid] + 1], [0]) for rid in live]
        for rid in live:
            at[rid] += 1
        done = [rid for rid in live if at[rid] == lens[rid]]
        steps.append({"entries": entries, "end": done})
        live = [rid for rid in live if rid not in done]
    second = ["e", "f"]
    steps += [{"entries": [(rid, prompts[rid][:34], list(range(34)))], "end": []} for rid in second]
    for i in range(34, 49):
        steps.append({"entries": [(rid, prompts[rid][i:i + 1], [0]) for rid in second], "end": second if i == 48 else []})
    runner = ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=16, num_pages=16,
                                        max_requests=4, max_seq_len=64)
    runner.max_graphs = 2
    seen = []
    real = runner._graph_step

    def spy(batch):
        out = real(batch)
        seen.append((batch.num_requests, sorted(runner._graphs)))
        return out
    runner._graph_step = spy
    ru.compare(ru.replay(runner, steps), want, tol_of(dtype), f"shapes that come and go {dtype}", skip)
    sizes = [n for n, _ in seen]
    assert sizes == [4] * 5 + [3] * 4 + [2] * 4 + [1] * 4 + [2] * 15
    # the third step of a shape captures it; never more than two graphs; the shape of four has gone by the end
    captured = [{k[0] for k in keys} for _, keys in seen]
    assert captured[1] == set() and captured[2] == {4} and all(len(c) <= 2 for c in captured)
    assert 4 not in captured[-1] and 2 in captured[-1]
    assert runner._graph_logits is not None and runner._graph_logits.shape == (4, cfg["vocab_size"])


def _edge(**over):
    base = {"architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "decoder_sparse_step": 1,
            "mlp_only_layers": [], "norm_topk_prob": False, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
            "max_position_embeddings": 1024, "use_sliding_window": False, "tie_word_embeddings": False,
            "intermediate_size": 40}
    base.update(over)
    return base


# the ends of what the architecture allows: one expert, one head, every expert chosen, a head of 256, a width of 16
# and of 1,000, a vocabulary of 17, a window of one key and one that no prompt reaches, six layers of three kinds
EDGE_CONFIGS = {
    "one_of_everything": (_edge(num_hidden_layers=2, hidden_size=16, num_attention_heads=1, num_key_value_heads=1,
                                head_dim=16, num_experts=1, num_experts_per_tok=1, moe_intermediate_size=8,
                                shared_expert_intermediate_size=0, vocab_size=17, use_sliding_window=True,
                                sliding_window=1, max_window_layers=1), 16, (2, 3, 64, 65)),
    "every_expert_chosen": (_edge(num_hidden_layers=2, hidden_size=1000, num_attention_heads=7, num_key_value_heads=1,
                                  head_dim=256, num_experts=7, num_experts_per_tok=7, moe_intermediate_size=200,
                                  shared_expert_intermediate_size=512, vocab_size=5003, norm_topk_prob=True,
                                  use_sliding_window=True, sliding_window=4096, max_window_layers=0,
                                  tie_word_embeddings=True, rms_norm_eps=1e-3), 64, (129, 300, 40)),
    "six_layers_three_kinds": (_edge(num_hidden_layers=6, hidden_size=320, num_attention_heads=16,
                                     num_key_value_heads=8, head_dim=32, num_experts=64, num_experts_per_tok=3,
                                     moe_intermediate_size=16, shared_expert_intermediate_size=8, vocab_size=64,
                                     decoder_sparse_step=3, mlp_only_layers=[2], intermediate_size=640, rope_theta=100.0,
                                     use_sliding_window=True, sliding_window=5, max_window_layers=3, qkv_bias=False),
                               16, (33, 257, 16, 90)),
    "window_of_two_in_pages_of_64": (_edge(num_hidden_layers=2, hidden_size=48, num_attention_heads=8,
                                           num_key_value_heads=8, head_dim=64, num_experts=4, num_experts_per_tok=3,
                                           moe_intermediate_size=384, shared_expert_intermediate_size=16,
                                           vocab_size=32000, use_sliding_window=True, sliding_window=2,
                                           max_window_layers=0), 64, (129, 500, 40)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(EDGE_CONFIGS))
def test_configurations_at_the_ends(tmp_path, name, dtype):
    """Whole, last tokens one by one, portions down to two tokens, and mixed, at the ends of the sizes."""
    from inferx_amd.engine.runner import ModelRunner
    cfg, page, lengths = EDGE_CONFIGS[name]
    tiny.make_folder(cfg, seed=3, out_dir=str(tmp_path), dtype=dtype)
    raw, weights = tiny.read_folder(str(tmp_path))
    prompts = {f"r{i}": tiny.random_tokens(n, cfg["vocab_size"], seed=50 + i) for i, n in enumerate(lengths)}
    want = ru.expected_logits(raw, weights, prompts)
    skip = ru.near_ties(raw, weights, prompts) if dtype == "bfloat16" else set()
    for how, steps in (("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 32)),
                       ("portions", ru.chunked(prompts, (256, 130, 2, 17, 200, 3))),
                       ("mixed", ru.mixed(prompts, seed=4, max_live=4))):
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=page, num_pages=4 * (512 // page + 2),
                                            max_requests=4, max_seq_len=1024)
        ru.compare(ru.replay(runner, steps), want, (ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL),
                   f"{name} {dtype} {how}", skip=skip)


@pytest.mark.parametrize("use_graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_entry_without_tokens_beside_one_with_two(folders, dtype, use_graphs):
    """A step may name a request that brings no token.  Beside a request that brings two, the step then has as
    many tokens as requests without being a step of one token each: it must not be taken for a decoding step
    (whose tiles and graphs assume row i = request i)."""
    from inferx_amd.engine.runner import ModelRunner
    name = "B"
    runner = ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=16, num_pages=64,
                                        max_requests=4, max_seq_len=1024, use_graphs=use_graphs)
    prompts = {k: v for k, v in list(prompts_for(name).items())[1:3]}
    (a, ta), (b, tb) = prompts.items()
    steps = [{"entries": [(a, ta[:9], list(range(9)))], "end": []},
             {"entries": [(b, tb[:20], list(range(20)))], "end": []},
             {"entries": [(a, [], []), (b, tb[20:22], [0, 1])], "end": []},       # 2 tokens, 2 requests
             {"entries": [(a, ta[9:11], [0, 1]), (b, [], [])], "end": []},
             {"entries": [(a, ta[11:12], [0]), (b, tb[22:23], [0])], "end": []},  # a true step of one token each
             {"entries": [(a, ta[12:], list(range(len(ta) - 12))), (b, tb[23:], list(range(len(tb) - 23)))],
              "end": [a, b]}]
    got = ru.replay(runner, steps)
    expected = {k: v for k, v in expected_for(folders, name, dtype).items() if k in prompts}
    ru.compare(got, expected, tol_of(dtype), f"empty entry {dtype} graphs={use_graphs}", ties_for(folders, name, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_giving_passed_pages_back_changes_no_logit(folders, name, dtype):
    """The windowed layers' pages with and without the early release: the kernels mask by the window either way,
    so the logits are the same bit for bit, while the pages held (summed over the steps) differ."""
    from inferx_amd.engine.runner import ModelRunner
    prompts = prompts_for(name)
    steps = ru.chunked(prompts) + ru.mixed({k + "m": v for k, v in prompts.items()}, seed=8, max_live=3)
    got, held = {}, {}
    for release in (True, False):
        runner = ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=16, num_pages=24,
                                            max_requests=4, max_seq_len=128, release_window_pages=release)
        windowed = [g for g, need in enumerate(runner.group_needs) if need.window > 0]
        assert windowed and runner.cache.groups[windowed[0]].release_passed is release
        held[release] = 0
        rows = {}
        for step in steps:
            rows.update(ru.replay(runner, [step]))
            held[release] += runner.cache.pools[windowed[0]].used_pages
        got[release] = rows
    assert held[True] < held[False]
    assert got[True].keys() == got[False].keys()
    for key in got[True]:
        assert torch.equal(got[True][key], got[False][key]), f"{key} differs with the release switched off"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_a_windowed_pool_sized_by_window_and_step(folders, name, dtype):
    """With the largest step promised, the windowed layers' pool holds window + step per request instead of a
    context's worth, pages are taken as the steps reach them, and no logit changes."""
    from inferx_amd.engine.runner import ModelRunner
    prompts = prompts_for(name)
    steps = ru.mixed(prompts, seed=8, max_live=3)           # no entry brings more than 33 tokens
    assert max(len(e[1]) for s in steps for e in s["entries"]) <= 33
    got = {}
    for cap in (None, 33):
        runner = ModelRunner.from_directory(folders[(name, dtype)], dtype=dtype, page_size=16, num_pages=24,
                                            max_requests=3, max_seq_len=128, max_step_tokens=cap)
        windowed = [g for g, need in enumerate(runner.group_needs) if need.window > 0][0]
        W = runner.group_needs[windowed].window
        want_pages = 24 if cap is None else 3 * (-(-(W + 33) // 16) + 2)
        assert runner.cache.pools[windowed].num_pages == want_pages < (25 if cap is None else 24)
        assert runner.pages[windowed]["k"].shape[1] == want_pages
        got[cap] = ru.replay(runner, steps)
        assert all(p.used_pages == 0 for p in runner.cache.pools)
    ru.compare(got[33], expected_for(folders, name, dtype), tol_of(dtype), f"windowed pool {name} {dtype}",
               ties_for(folders, name, dtype))
    for key in got[None]:
        assert torch.equal(got[None][key], got[33][key]), f"{key} differs with the smaller pool"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [4, 8, 24, 48, 128])
def test_pages_of_other_sizes(folders, page_size, dtype):
    """Pages of 4, 8, 24, 48 and 128 tokens (the command line takes any positive `--block-size`, reference
    src/support/options.cc:47-174): configuration B, with dense and expert layers, full and windowed attention (a
    window of 16, so pages of 4 and 8 are given back while a request runs), the four ways.  A page that is no
    multiple of 16 sends bfloat16 attention to the plain kernel, one that is no power of two keeps portions off the
    LDS-sharing kernel; the logits are the plain implementation's either way."""
    name = "B"
    prompts = prompts_for(name)
    expected, ties = expected_for(folders, name, dtype), ties_for(folders, name, dtype)
    max_tokens = 192 if page_size <= 64 else 256
    pages = max_tokens // page_size
    for how, steps in [("whole", ru.whole(prompts)), ("tail", ru.tail_decoded(prompts, 32)),
                       ("chunked", ru.chunked(prompts)),
                       ("mixed", ru.mixed(prompts, seed=8, max_tokens=max_tokens, round_to=max(64, page_size)))]:
        runner = make_runner(folders, name, dtype, num_pages=pages, page_size=page_size)
        assert runner.page_size == page_size and runner.pages[0]["k"].shape[3] == page_size
        owners = {}
        got = ru.replay(runner, steps, page_owners=owners)
        ru.compare(got, expected, tol_of(dtype), f"pages of {page_size}, {how} {dtype}", ties)
        assert all(p.used_pages == 0 for p in runner.cache.pools)
        if how == "mixed":
            assert any(len(rids) > 1 for rids in owners.values()), "no page was used again"
        if how == "tail":
            assert runner._graphs
