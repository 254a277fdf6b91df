"""Generation through the entry points: the Python engine, the command line and the replay
program, against the plain implementation; long decoding; the first tokens of a sequence;
what happens when pages run out."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_model as pm
import replay_util as ru
import tiny

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_greedy(cfg, weights, prompt, steps):
    seq, margins = list(prompt), []
    for _ in range(steps):
        logits = pm.forward(cfg, weights, seq)[-1]
        top2 = torch.topk(logits, 2).values
        margins.append(float(top2[0] - top2[1]) / float(logits.abs().max()))
        seq.append(pm.greedy(logits))
    return seq[len(prompt):], margins


def check_greedy(got, want, margins, exact):
    for i, (g, w, m) in enumerate(zip(got, want, margins)):
        if g != w:
            assert not exact and m < 2e-2, f"token {i}: got {g}, plain implementation {w} (margin {m:.2e})"
            return  # after a near-tie the two continuations legitimately differ
    assert len(got) == len(want)


@pytest.mark.parametrize("name,dtype,lengths,steps", [("A", "float32", (5, 9, 17), 8), ("B", "float32", (7, 23, 40), 12),
                                                      ("A", "bfloat16", (5, 9, 17), 8), ("B", "bfloat16", (7, 23, 40), 12)])
def test_greedy_generation_through_the_python_entry_point(tmp_path, name, dtype, lengths, steps):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIGS[name], 31, str(tmp_path), dtype)
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 40 + n) for n in lengths]
    # portions of 8 tokens (the second configuration's workload), three requests at a time
    engine = LLMEngine(str(tmp_path), dtype, max_num_seqs=3, max_model_len=128, max_num_batched_tokens=8,
                       num_gpu_blocks_override=24)
    got = engine.generate(prompts, SamplingParams(max_tokens=steps))
    for p, g in zip(prompts, got):
        want, margins = plain_greedy(cfg, weights, p, steps)
        check_greedy(g, want, margins, exact=dtype == "float32")
    assert engine.stats.tokens_out == steps * len(prompts)
    assert all(pool.used_pages == 0 for pool in engine.runner.cache.pools)


def test_temperature_sampling_is_seeded_and_in_the_support(tmp_path):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_B, 32, str(tmp_path), "float32", std_scale=6.0)  # peaked enough for small supports
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 50 + n) for n in (7, 23, 40)]
    params = SamplingParams(max_tokens=12, temperature=0.7, top_k=6, seed=99)
    runs = []
    for _ in range(2):
        engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=3, max_model_len=128, max_num_batched_tokens=8,
                           num_gpu_blocks_override=24)
        runs.append(engine.generate(prompts, params))
    assert runs[0] == runs[1]  # a pinned seed reproduces
    for p, out in zip(prompts, runs[0]):
        seq = list(p)
        for tok in out:
            logits = pm.forward(cfg, weights, seq)[-1]
            assert tok in pm.sampling_support(logits, 0.7, top_k=6)
            seq.append(tok)
    other = LLMEngine(str(tmp_path), "float32", max_num_seqs=3, max_model_len=128, num_gpu_blocks_override=24)
    assert other.generate(prompts, SamplingParams(max_tokens=12, temperature=0.7, top_k=6, seed=100)) != runs[0]


def test_logprobs_through_the_engine(tmp_path):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 39, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompt = tiny.random_tokens(11, cfg["vocab_size"], 71)
    engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=2, max_model_len=64, num_gpu_blocks_override=8)
    out = engine.generate([prompt], SamplingParams(max_tokens=4, want_logprobs=True, top_logprobs=3))[0]
    lps = engine.last_completions[0].logprobs
    assert len(lps) == 4
    seq = list(prompt)
    for tok, (lp, top) in zip(out, lps):
        want = torch.log_softmax(pm.forward(cfg, weights, seq)[-1], -1)
        assert abs(lp - float(want[tok])) < 1e-4
        assert [t for t, _ in top] == torch.topk(want, 3).indices.tolist() and top[0][0] == tok  # greedy: chosen = top
        assert max(abs(v - float(want[t])) for t, v in top) < 1e-4
        seq.append(tok)


def test_preempted_generation_equals_unpreempted(tmp_path):
    """So few pages that running requests are preempted and recomputed: same tokens (reference:
    tests/unit/scheduler_test.cc:742-812)."""
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 33, str(tmp_path), "float32")
    cfg, _ = tiny.read_folder(str(tmp_path))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 60 + n) for n in (20, 25, 30)]
    params = [SamplingParams(max_tokens=40, temperature=0.8, seed=i) for i in range(3)]
    roomy = LLMEngine(str(tmp_path), "float32", max_num_seqs=3, max_model_len=128, num_gpu_blocks_override=24)
    tight = LLMEngine(str(tmp_path), "float32", max_num_seqs=3, max_model_len=128, num_gpu_blocks_override=9)
    a, b = roomy.generate(prompts, params), tight.generate(prompts, params)
    assert roomy.stats.preemptions == 0 and tight.stats.preemptions > 0
    assert a == b
    # The rows' settings and the numbers of their next draws stay on the device while the same requests sample (the
    # kernel moves the numbers on): they went up when a prompt had been read or a request had ended, not at each of
    # the 40 steps; and a third run that brings them up at every step draws the same tokens.
    assert roomy.sampler.uploads <= 8 < roomy.stats.steps
    naive = LLMEngine(str(tmp_path), "float32", max_num_seqs=3, max_model_len=128, num_gpu_blocks_override=24)
    launch = naive.sampler.launch

    def forgetful(logits, rows):
        naive.sampler._resident = None
        return launch(logits, rows)
    naive.sampler.launch = forgetful
    assert naive.generate(prompts, params) == a and naive.sampler.uploads >= 40


def test_stop_token_and_context_limit(tmp_path):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 34, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompt = tiny.random_tokens(6, cfg["vocab_size"], 70)
    want, _ = plain_greedy(cfg, weights, prompt, 6)
    engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=2, max_model_len=32, num_gpu_blocks_override=8)
    out = engine.generate([prompt], SamplingParams(max_tokens=20, stop_tokens=[want[3]]), with_reasons=True)
    first_stop = want.index(want[3])
    assert out[0] == (want[:first_stop + 1], "stop_token")
    out = engine.generate([prompt], SamplingParams(max_tokens=100), with_reasons=True)
    assert out[0][1] == "context_limit" and len(out[0][0]) == 32 - 6 + 1


def test_end_of_sequence_ids_of_the_model_stop_a_request_unless_it_ignores_them(tmp_path):
    """config.json's eos_token_id joins every request's stop tokens (reference: src/engine/engine.cc:819-823)."""
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 34, str(tmp_path / "plain"), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path / "plain"))
    prompt = tiny.random_tokens(6, cfg["vocab_size"], 70)
    want, _ = plain_greedy(cfg, weights, prompt, 8)
    eos = want[2]
    first = want.index(eos)
    tiny.make_folder({**tiny.CONFIG_A, "eos_token_id": eos}, 34, str(tmp_path / "eos"), "float32")  # same weights
    engine = LLMEngine(str(tmp_path / "eos"), "float32", max_num_seqs=2, max_model_len=32, num_gpu_blocks_override=8)
    out = engine.generate([prompt], SamplingParams(max_tokens=8), with_reasons=True)
    assert out[0] == (want[:first + 1], "stop_token")
    out = engine.generate([prompt], SamplingParams(max_tokens=8, ignore_eos=True), with_reasons=True)
    assert out[0] == (want, "max_tokens")
    # before min_tokens the stop tokens are masked out of the choice: another token is taken in their place
    got = engine.generate([prompt], SamplingParams(max_tokens=8, min_tokens=first + 2))[0]
    assert got[:first] == want[:first] and eos not in got[:first + 2] and len(got) >= first + 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(tmp_path, dtype):
    """300 tokens one by one after a two-token start (graphs, page edges, the window), and every
    first position of a sequence, against the plain implementation."""
    from inferx_amd.engine.runner import ModelRunner
    tiny.make_folder(tiny.CONFIG_B, 35, str(tmp_path), dtype)
    cfg, weights = tiny.read_folder(str(tmp_path))
    toks = tiny.random_tokens(250, cfg["vocab_size"], 80)
    expected = {"r": pm.forward(cfg, weights, toks)}
    runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=16, max_requests=2,
                                        max_seq_len=256)
    steps = [{"entries": [("r", toks[:2], [0, 1])], "end": []}]
    steps += [{"entries": [("r", toks[i:i + 1], [0])], "end": []} for i in range(2, 250)]
    got = ru.replay(runner, steps)
    ru.compare(got, expected, ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL, f"long decode {dtype}")
    assert runner.use_graphs and len(runner._graphs) >= 2  # captured steps were replayed, over several buckets


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_whose_keys_are_cut_into_slices(tmp_path, dtype, monkeypatch):
    """A prompt read in portions on top of a growing context, with the rule that cuts a portion's keys into slices
    (a workgroup each; from about 6,000 keys on) brought down to 512 keys so that the plain implementation can
    follow; then tokens one by one (keys in several slices there too), on layers with and without a window."""
    from inferx_amd import ops
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts import attention
    monkeypatch.setattr(attention, "PREFILL_SLICED_MIN_ROUNDS", 8)
    monkeypatch.setattr(attention, "PREFILL_SLICE_ROUNDS", 2)
    monkeypatch.setattr(attention, "PREFILL_MIN_WORKGROUPS", 0)
    sliced = []
    real = ops.attention_prefill

    def spy(*args, **kwargs):
        sliced.append(args[11] if len(args) > 11 else kwargs.get("n_splits", 1))
        return real(*args, **kwargs)
    monkeypatch.setattr(ops, "attention_prefill", spy)
    raw = dict(tiny.CONFIG_B, max_position_embeddings=2048)
    tiny.make_folder(raw, 37, str(tmp_path), dtype)
    cfg, weights = tiny.read_folder(str(tmp_path))
    toks = tiny.random_tokens(1100, cfg["vocab_size"], 82)
    whole = pm.forward(cfg, weights, toks)
    runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=72, max_requests=2,
                                        max_seq_len=1152)
    steps, at = [], 0
    for n in (384, 384, 320):
        steps.append({"entries": [("r", toks[at:at + n], [0, 1, n // 2, n - 2, n - 1])], "end": []})
        at += n
    steps += [{"entries": [("r", toks[i:i + 1], [0])], "end": []} for i in range(at, len(toks))]
    got = ru.replay(runner, steps)
    assert len(got) == 15 + 12
    assert dtype == "float32" or any(n > 1 for n in sliced), "no portion's keys were cut into slices"
    scale = float(whole.abs().max())
    worst = max(float((row.double() - whole[pos]).abs().max()) / scale for (_, pos), row in got.items())
    assert worst < (ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL), f"{dtype}: {worst:.3e} of the largest logit"


def test_a_context_of_thousands_of_tokens_in_both_types(tmp_path, monkeypatch):
    """9,000 tokens, too many for the plain implementation of the whole model.  Every call of the attention part,
    in both runs, is compared with float64 attention over the keys and values that the cache holds at that moment
    (read back through the block table): portions of 2,048 on up to 8,192 keys, keys cut into slices for portions
    and for single tokens, a captured graph for a context of thousands, full and windowed layers.  Beyond that the
    two kernel families check each other, engine against engine: the same bfloat16 weights run in float32 (plain
    kernels) and in bfloat16 (matrix-core kernels), and the logits at the portions' ends and of the last tokens
    agree within the bfloat16 bound."""
    import attention_util as au
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.parts.attention import PagedAttention
    raw = dict(tiny.CONFIG_B, max_position_embeddings=16384)
    tiny.make_folder(raw, 38, str(tmp_path), "bfloat16")
    # (random weights attend almost evenly, and one lost slice of 9,000 keys would hardly show: with the query and
    # key weights scaled up the scores are peaked)
    from safetensors.torch import save_file
    _, weights = tiny.read_folder(str(tmp_path))
    for k in weights:
        if "q_proj.weight" in k or "k_proj.weight" in k:
            weights[k] = weights[k] * 8.0
    save_file(weights, os.path.join(str(tmp_path), "model.safetensors"))
    toks = tiny.random_tokens(9006, raw["vocab_size"], 83)
    steps, at = [], 0
    for n in (2048, 2048, 2048, 2048, 808):
        steps.append({"entries": [("r", toks[at:at + n], [n - 1])], "end": []})
        at += n
    steps += [{"entries": [("r", toks[i:i + 1], [0])], "end": []} for i in range(at, len(toks))]
    real_attend = PagedAttention.attend
    checked = {"calls": 0, "worst": 0.0, "windowed": 0, "no_host": 0}
    shape = {}  # the step's host arrays, set before each step below (a captured step's context has none)

    def attend(self, ctx, q, cache, out):
        real_attend(self, ctx, q, cache, out)
        if torch.cuda.is_current_stream_capturing():
            return  # (a recording runs nothing; the warm-up run before it was checked)
        want = au.attention_from_cache(q, cache.k, cache.v, ctx.block_tables[cache.group], shape["q_start"],
                                       shape["seq_lens"], self.scale, self.window)
        checked["calls"] += 1
        checked["windowed"] += self.window > 0
        checked["no_host"] += ctx.host is None
        checked["worst"] = max(checked["worst"], au.rel_err(out, want))
    monkeypatch.setattr(PagedAttention, "attend", attend)
    got = {}
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_directory(str(tmp_path), dtype=dtype, page_size=16, num_pages=576, max_requests=2,
                                            max_seq_len=9216)
        runner.capture_after = 2
        real_step = runner.step

        def step(batch, real_step=real_step):
            shape["q_start"], shape["seq_lens"] = batch.q_start.copy(), batch.seq_lens.copy()
            return real_step(batch)
        runner.step = step
        checked.update(calls=0, worst=0.0, windowed=0, no_host=0)
        got[dtype] = ru.replay(runner, steps)
        assert len(got[dtype]) == 5 + 6
        layers = raw["num_hidden_layers"]
        assert checked["calls"] >= layers * (5 + 2) and checked["windowed"] >= 2 * (5 + 2)
        assert checked["worst"] < (1e-5 if dtype == "float32" else 1.5e-2), \
            f"{dtype}: an attention call differs from float64 attention by {checked['worst']:.3e}"
        if dtype == "bfloat16":
            assert runner._graphs and checked["no_host"] >= layers  # the warm-up run of a recording was checked too
    scale = max(float(row.abs().max()) for row in got["float32"].values())
    errs = {pos: float((got["bfloat16"][(rid, pos)].double() - row.double()).abs().max()) / scale
            for (rid, pos), row in got["float32"].items()}
    assert max(errs.values()) < ru.BF16_TOL, f"the two runs differ: {errs}"


def test_far_key_and_window_edge_show_in_the_logits(tmp_path):
    """Random weights attend almost uniformly and would hide a lost key.  With attention weights scaled up the
    scores are peaked, so a key lost at a page edge, a split boundary or the window's edge changes the logits."""
    from inferx_amd.engine.runner import ModelRunner
    raw = dict(tiny.CONFIG_B, max_position_embeddings=512)
    tiny.make_folder(raw, 36, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    from safetensors.torch import save_file
    for k in weights:
        if "q_proj.weight" in k or "k_proj.weight" in k:
            weights[k] = weights[k] * 12.0
    save_file(weights, os.path.join(str(tmp_path), "model.safetensors"))
    toks = tiny.random_tokens(300, cfg["vocab_size"], 81)
    whole = pm.forward(cfg, weights, toks)
    # the plain implementation itself is sensitive here: dropping the oldest key of the window changes the result
    assert float((pm.forward(dict(cfg, sliding_window=15), weights, toks)[-1] - whole[-1]).abs().max()) > \
        1e-3 * float(whole.abs().max())
    runner = ModelRunner.from_directory(str(tmp_path), dtype="float32", page_size=16, num_pages=24, max_requests=2,
                                        max_seq_len=384)
    prompts = {"r": toks}
    for steps in (ru.whole(prompts), ru.chunked(prompts, sizes=(33, 2, 64, 17, 100)), ru.tail_decoded(prompts, 40)):
        ru.compare(ru.replay(runner, steps), {"r": whole}, ru.FP32_TOL, "peaked attention")


def test_enforce_eager_gives_the_same_tokens_without_graphs(tmp_path):
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 41, str(tmp_path), "bfloat16")
    cfg, _ = tiny.read_folder(str(tmp_path))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 70 + n) for n in (5, 18)]
    outs = []
    for eager in (False, True):
        engine = LLMEngine(str(tmp_path), "bfloat16", max_num_seqs=2, max_model_len=64, num_gpu_blocks_override=12,
                           enforce_eager=eager)
        assert engine.runner.use_graphs == (not eager)
        outs.append(engine.generate(prompts, SamplingParams(max_tokens=10)))
        assert bool(engine.runner._graphs) == (not eager)
    assert outs[0] == outs[1]


def test_planning_the_next_step_ahead_changes_no_output(tmp_path):
    """The engine plans and lays out the next step while the device runs this one.  With it and without it: the
    same tokens and reasons, under stop tokens, min_tokens, seeded temperature sampling with cut-offs, penalties
    and scarce pages (float32, so that a change of batch composition cannot flip a draw)."""
    import random
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_B, 41, str(tmp_path), "float32")
    vocab = tiny.CONFIG_B["vocab_size"]
    rnd = random.Random(5)
    prompts = [tiny.random_tokens(rnd.randint(1, 50), vocab, seed=300 + i) for i in range(9)]
    params = [SamplingParams(max_tokens=rnd.randint(1, 18), temperature=rnd.choice([0.0, 0.7, 1.3]),
                             top_p=rnd.choice([1.0, 0.9]), top_k=rnd.choice([0, 5]), seed=rnd.randrange(1000),
                             stop_tokens=[rnd.randrange(vocab) for _ in range(rnd.choice([0, 20, 60]))],
                             min_tokens=rnd.choice([0, 2]), repetition_penalty=rnd.choice([1.0, 1.2]),
                             presence_penalty=rnd.choice([0.0, 0.5])) for _ in prompts]
    outs = []
    for ahead in (False, True):
        engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=4, max_model_len=80, max_num_batched_tokens=48,
                           num_gpu_blocks_override=9)
        engine.plan_ahead = ahead
        outs.append(engine.generate(prompts, params, with_reasons=True))
        assert engine.runner.cache.pools[0].used_pages == 0
    assert outs[0] == outs[1]
    assert any(r == "stop_token" for _, r in outs[1]) and any(r == "max_tokens" for _, r in outs[1])


def test_command_line(tmp_path):
    tiny.make_folder(tiny.CONFIG_A, 37, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompt = tiny.random_tokens(9, cfg["vocab_size"], 90)
    want, _ = plain_greedy(cfg, weights, prompt, 5)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "inferx-generate"), "--model", str(tmp_path), "--dtype", "float32",
           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5", "--max-model-len", "64",
           "--num-gpu-blocks-override", "8", "--max-num-seqs", "2"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["output_token_ids"] == want and rec["finish_reason"] == "max_tokens"
    more = subprocess.run(cmd + ["--logprobs", "2", "--ignore-eos", "--min-tokens", "1"], capture_output=True, text=True,
                          timeout=300)
    assert more.returncode == 0, more.stderr
    rec = json.loads(more.stdout.strip().splitlines()[-1])
    assert rec["output_token_ids"] == want and len(rec["logprobs"]) == 5
    assert all(len(lp["top"]) == 2 and lp["logprob"] <= 0.0 and lp["top"][0][1] >= lp["top"][1][1] for lp in rec["logprobs"])
    assert [lp["top"][0][0] for lp in rec["logprobs"]] == want  # greedy: the chosen token is the most probable one
    bad = subprocess.run(cmd[:2] + ["--no-such-flag"], capture_output=True, text=True, timeout=60)
    assert bad.returncode == 2
    missing = subprocess.run(cmd[:2] + ["--model", os.path.join(str(tmp_path), "nothing"), "--prompt-ids", "1"],
                             capture_output=True, text=True, timeout=120)
    assert missing.returncode == 1 and "config.json" in missing.stderr


def test_command_line_sizes_the_cache_by_memory_and_dumps_logits(tmp_path):
    """The command line without --num-gpu-blocks-override (the pool is sized from the memory that is free), with
    --kv-cache-memory-bytes, and --dump-logits: the reference's logits file, against the plain implementation."""
    import struct
    model = tmp_path / "m"
    tiny.make_folder(tiny.CONFIG_B, 41, str(model), "float32")
    cfg, weights = tiny.read_folder(str(model))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 60 + n) for n in (9, 40)]
    want = [plain_greedy(cfg, weights, p, 4)[0] for p in prompts]
    base = [sys.executable, os.path.join(ROOT, "bin", "inferx-generate"), str(model), "--dtype", "float32",
            "--max-tokens", "4", "--max-model-len", "96", "--max-num-seqs", "2", "--max-num-batched-tokens", "16"]
    for p in prompts:
        base += ["--prompt-ids", ",".join(map(str, p))]
    dump = tmp_path / "logits.bin"
    out = subprocess.run(base + ["--dump-logits", str(dump), "--log-level", "info", "--log-json"], capture_output=True,
                         text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    sized = [json.loads(l) for l in out.stderr.splitlines() if l.startswith("{")]
    assert any(r["level"] == "info" and "pages of 16 tokens" in r["message"] for r in sized), out.stderr
    recs = [json.loads(l) for l in out.stdout.strip().splitlines()]
    assert [r["output_token_ids"] for r in recs] == want
    raw = dump.read_bytes()
    at = 0
    for p in prompts:
        assert raw[at:at + 4] == b"IXRL"
        version, tokens, vocab = struct.unpack_from("<III", raw, at + 4)
        assert (version, tokens, vocab) == (1, len(p), cfg["vocab_size"])
        assert list(struct.unpack_from(f"<{tokens}i", raw, at + 16)) == p
        at += 16 + 4 * tokens
        rows = torch.from_numpy(np.frombuffer(raw, dtype="<f4", count=tokens * vocab, offset=at).copy()).view(tokens, vocab)
        at += 4 * tokens * vocab
        expect = pm.forward(cfg, weights, p)
        assert float((rows.double() - expect).abs().max()) <= ru.FP32_TOL * float(expect.abs().max())
    assert at == len(raw)
    # an explicit budget in bytes: 6 pages of 16 tokens are just enough for one sequence of 96
    page_bytes = 16 * 4 * 2 * 1 * 32 * 4  # tokens x layers x (k, v) x kv heads x head size x float32
    sized = subprocess.run(base + ["--kv-cache-memory-bytes", str(6 * page_bytes)], capture_output=True, text=True,
                           timeout=300)
    assert sized.returncode == 0, sized.stderr
    assert [json.loads(l)["output_token_ids"] for l in sized.stdout.strip().splitlines()] == want
    small = subprocess.run(base + ["--kv-cache-memory-bytes", str(5 * page_bytes)], capture_output=True, text=True,
                           timeout=300)
    assert small.returncode == 1 and "--kv-cache-memory-bytes" in small.stderr and "--max-model-len" in small.stderr


def test_generation_with_a_small_token_budget_and_windowed_layers(tmp_path):
    """The engine promises its token budget to the cache: the windowed layers' pool is sized by window + budget,
    prompts longer than that pool run through it in portions, and the tokens are the plain implementation's."""
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_B, 47, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=2, max_model_len=192, max_num_batched_tokens=16,
                       num_gpu_blocks_override=24)
    pools = engine.runner.cache.pools
    assert [p.num_pages for p in pools] == [24, 2 * (2 + 2)]  # window 16, budget 16, pages of 16, two requests
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 70 + n) for n in (150, 90, 33)]
    got = engine.generate(prompts, SamplingParams(max_tokens=5))
    for p, out in zip(prompts, got):
        assert out == plain_greedy(cfg, weights, p, 5)[0]
    assert all(p.used_pages == 0 for p in pools)


def test_a_prompt_larger_than_the_pool_ends_out_of_memory(tmp_path):
    """Two pages and a prompt of 40: the request ends out_of_memory at once and the next one runs; the loop does
    not wait for pages that nobody will give back."""
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.sampling import SamplingParams
    tiny.make_folder(tiny.CONFIG_A, 43, str(tmp_path), "float32")
    cfg, weights = tiny.read_folder(str(tmp_path))
    engine = LLMEngine(str(tmp_path), "float32", max_num_seqs=2, max_model_len=64, num_gpu_blocks_override=2)
    big, small = tiny.random_tokens(40, cfg["vocab_size"], 1), tiny.random_tokens(9, cfg["vocab_size"], 2)
    got = engine.generate([big, small], SamplingParams(max_tokens=3), with_reasons=True)
    assert got[0] == ([], "out_of_memory")
    assert got[1] == (plain_greedy(cfg, weights, small, 3)[0], "max_tokens")
    assert engine.runner.cache.pools[0].used_pages == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    """bin/trace_run as a user calls it: steps on standard input, logits in files, `done <step>` per step."""
    model = tmp_path / "model"
    out_dir = tmp_path / "out"
    tiny.make_folder(tiny.CONFIG_B, 38, str(model), dtype)
    cfg, weights = tiny.read_folder(str(model))
    prompts = {f"r{i}": tiny.random_tokens(n, cfg["vocab_size"], 95 + i) for i, n in enumerate((40, 70, 23, 55, 64))}
    steps = ru.mixed(prompts, seed=9, max_live=4, max_tokens=256)
    lines, wanted = [], []
    fed = {rid: 0 for rid in prompts}
    for i, st in enumerate(steps):
        entries = []
        for rid, toks, want in st["entries"]:
            want = want if (i + len(toks)) % 3 else want[::2]  # not every place is asked for
            entries.append({"id": rid, "tokens": toks, "want": want})
            wanted.append((i, [(rid, fed[rid] + w) for w in want]))
            fed[rid] += len(toks)
        lines.append(json.dumps({"step": i, "entries": entries, "end": st["end"]}))
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(model), "--dtype", dtype, "--out",
                           str(out_dir), "--max-tokens", "256"], input="\n".join(lines) + "\n", capture_output=True,
                          text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for i in range(len(steps)) for w in ("done", str(i))]
    got = {}
    by_step = {}
    for i, keys in wanted:
        by_step.setdefault(i, []).extend(keys)
    for i, keys in by_step.items():
        path = out_dir / f"{i}.f32"
        if not keys:
            assert not path.exists()
            continue
        rows = np.fromfile(path, dtype="<f4").reshape(len(keys), cfg["vocab_size"])
        for key, row in zip(keys, rows):
            got[key] = torch.from_numpy(row.copy())
    expected = ru.expected_logits(cfg, weights, prompts)
    tol = ru.FP32_TOL if dtype == "float32" else ru.BF16_TOL
    scale = max(float(e.abs().max()) for e in expected.values())
    assert len(got) > 100
    for (rid, pos), row in got.items():
        err = float((row.double() - expected[rid][pos]).abs().max()) / scale
        assert err <= tol, f"request {rid} position {pos}: error {err:.2e}"


def test_one_token_steps_give_the_same_bits_before_and_after_their_shape_is_recorded(tmp_path):
    """A shape of (requests, context bucket) runs kernel by kernel until it has come `capture_after` times and
    from a graph afterwards.  Both ways plan with the bucket (520 keys: eight slices of the keys either way, where the
    true length alone would give four), so a request's bfloat16 logits do not depend on what the engine has
    served before."""
    from inferx_amd.engine.runner import ModelRunner
    tiny.make_folder(dict(tiny.CONFIG_A, max_position_embeddings=1024), 5, str(tmp_path), "bfloat16")
    toks = tiny.random_tokens(530, 256, 3)
    got = {}
    for after in (1, 3, 10 ** 6):
        runner = ModelRunner.from_directory(str(tmp_path), dtype="bfloat16", page_size=16, num_pages=40,
                                            max_requests=1, max_seq_len=640)
        runner.capture_after = after
        runner.add_request("a")
        runner.run_entries([("a", toks[:518], [])])
        rows = [runner.run_entries([("a", toks[i:i + 1], [0])]).clone() for i in range(518, 530)]
        assert bool(runner._graphs) == (after < 10 ** 6)
        got[after] = torch.cat(rows)
    assert torch.equal(got[1], got[3]) and torch.equal(got[1], got[10 ** 6])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_with_pages_of_eight_tokens(tmp_path, dtype):
    """`--block-size 8` through the command line: greedy tokens of the plain implementation (configuration B: the
    window of 16 passes two pages of eight while a request runs)."""
    tiny.make_folder(tiny.CONFIG_B, 43, str(tmp_path), dtype)
    cfg, weights = tiny.read_folder(str(tmp_path))
    prompts = [tiny.random_tokens(n, cfg["vocab_size"], 70 + n) for n in (11, 37)]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "inferx-generate"), str(tmp_path), "--dtype", dtype,
           "--max-tokens", "6", "--max-model-len", "64", "--max-num-seqs", "2", "--block-size", "8",
           "--num-gpu-blocks-override", "16", "--log-level", "info"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert "of 8 tokens" in out.stderr
    recs = [json.loads(l) for l in out.stdout.strip().splitlines()]
    for rec, p in zip(recs, prompts):
        want, margins = plain_greedy(cfg, weights, p, 6)
        # (bfloat16 may leave the plain implementation's path only where its two best logits nearly tie)
        check_greedy(rec["output_token_ids"], want, margins, exact=dtype == "float32")
