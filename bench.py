"""Decode and prefill throughput at the Qwen1.5-MoE-A2.7B shape, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of the whole batch through the engine (scheduler,
batch layout, upload, every kernel, greedy choice of the next tokens).  Prints ONE
JSON line: decoded tokens a second at the default batch (with the smallest and the
median time of single steps), the prefill of one 2,048-token prompt, the decode
step's HBM roofline fraction, and decode at batch 1 and 64.  Fractions are given
against the published peaks and against what two probe kernels measure on this
machine at the start of the run (a pure read of 4 GiB, pure matrix-core
products).  One GPU only.

Two further workloads at the Qwen2-57B-A14B shape, each with a JSON line of the same form:

    python bench.py --workload mixed [--layers L]   # 32 decodes at a context of 4,096 beside 2 prompt portions of 512
    python bench.py --workload long [--layers L]    # batch 8, prompts of 16,384 to 32,000 tokens in portions of
                                                    # 2,048, then --steps decode steps (default there: 256)

and a small mixed step at the Qwen1.5-MoE-A2.7B shape, which is launched kernel by kernel (only steps of one token
per request are replayed from HIP graphs): under `rocprofv3 --kernel-trace` it shows whether such steps wait for
the host:

    python bench.py --workload mixed-small          # 8 decodes at a context of 2,048 beside 1 prompt portion of 64

and a prompt portion on top of a context at either shape (chunked prefill under a token budget), through the step
function:

    python bench.py --workload portion --shape a27b|57b --prefill-tokens N --prefill-context C [--layers L]

and a whole batch through the engine's loop (scheduler, portions, decode graphs as they come, sampling) at the same
shape:

    python bench.py --workload offline              # 96 requests of 5 to 3,000 prompt tokens and 4 to 120 generated,
                                                    # 64 at a time, 4,096 tokens a step; with --scarce so few pages
                                                    # that sequences are preempted
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen1.5-MoE-A2.7B's sizes
SHAPE = {
    "architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": 24, "hidden_size": 2048,
    "num_attention_heads": 16, "num_key_value_heads": 16, "head_dim": 128, "num_experts": 60,
    "num_experts_per_tok": 4, "moe_intermediate_size": 1408, "shared_expert_intermediate_size": 5632,
    "intermediate_size": 5632, "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 8192,
    "use_sliding_window": False, "tie_word_embeddings": False,
}
# Qwen2-57B-A14B's sizes
SHAPE_57B = {
    "architectures": ["Qwen2MoeForCausalLM"], "num_hidden_layers": 28, "hidden_size": 3584,
    "num_attention_heads": 28, "num_key_value_heads": 4, "head_dim": 128, "num_experts": 64,
    "num_experts_per_tok": 8, "moe_intermediate_size": 2560, "shared_expert_intermediate_size": 20480,
    "intermediate_size": 18944, "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 32768,
    "use_sliding_window": False, "tie_word_embeddings": False,
}
CONTEXT = 4096
PROMPT = 2048
PAGE = 16
PEAK_HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def decode_bytes(cfg, batch, context, elt, distinct=None):
    """Bytes one decode step has to read: every weight it uses once, and the cache of the live requests.
    `distinct`: experts that a step's tokens choose, per layer (measured); without it what an even router gives."""
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    if distinct is None:
        distinct = E * (1.0 - (1.0 - k / E) ** batch)  # expected number of experts a batch touches
    per_layer = (qd + 2 * kvd) * H + (qd + 2 * kvd) + H * qd + 2 * H  # attention + norms
    per_layer += E * H + distinct * 3 * mi * H + 3 * si * H + H      # router, routed, shared, shared gate
    weights = L * per_layer + H + cfg.vocab_size * H + batch * H     # final norm, head, embedding rows
    cache = L * 2 * kvd * context * batch
    return (weights + cache) * elt


def prefill_flops(cfg, tokens):
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    per_token = (qd + 2 * kvd) * H + H * qd + E * H + k * 3 * mi * H + 3 * si * H + H
    linear = 2.0 * tokens * L * per_token + 2.0 * cfg.vocab_size * H  # head on the last row only
    attention = L * 2.0 * 2.0 * qd * tokens * (tokens + 1) / 2.0     # causal half of QK^T and PV
    return linear + attention


def experts_hit(run_step, runner, steps=2):
    """How many experts the tokens of a step really choose, per layer: `steps` steps run without graphs, the
    grouping's offsets read back."""
    import torch
    from inferx_amd import ops
    seen, hit, graphs = [], [], runner.use_graphs
    real = ops.moe_route_dispatch, ops.moe_dispatch

    def spy_small(*a, **k):
        real[0](*a, **k)
        seen.append(a[8])

    def spy_wide(topk_e, offsets, *a, **k):
        real[1](topk_e, offsets, *a, **k)
        seen.append(offsets)
    try:
        runner.use_graphs = False
        ops.moe_route_dispatch, ops.moe_dispatch = spy_small, spy_wide
        for _ in range(steps):
            seen.clear()
            run_step()
            torch.cuda.synchronize()  # (the offsets of a layer are a buffer of their own until the step ends)
            hit += [int(((o[1:] - o[:-1]) > 0).sum()) for o in seen]
    finally:
        runner.use_graphs = graphs
        ops.moe_route_dispatch, ops.moe_dispatch = real
    return sum(hit) / len(hit) if hit else None


def step_bytes(cfg, tokens, cache_tokens, elt, distinct=None):
    """Bytes a step of `tokens` tokens has to read: every weight it uses once, and `cache_tokens` of cache.
    `distinct`: experts that the step's tokens choose, per layer (measured); without it what an even router gives."""
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    if distinct is None:
        distinct = E * (1.0 - (1.0 - k / E) ** tokens)
    per_layer = (qd + 2 * kvd) * H + (qd + 2 * kvd) + H * qd + 2 * H + E * H + distinct * 3 * mi * H + 3 * si * H + H
    return (L * per_layer + H + cfg.vocab_size * H + L * 2 * kvd * cache_tokens) * elt


def linear_flops(cfg, tokens, head_rows):
    H, L = cfg.hidden_size, cfg.num_hidden_layers
    qd, kvd = cfg.q_dim, cfg.kv_dim
    E, k, mi, si = cfg.num_experts, cfg.num_experts_per_tok, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    per_token = (qd + 2 * kvd) * H + H * qd + E * H + k * 3 * mi * H + 3 * si * H + H
    return 2.0 * tokens * L * per_token + 2.0 * head_rows * cfg.vocab_size * H


def attention_flops(cfg, new, before):
    """QK^T and PV of `new` tokens that follow `before` cached ones (causal)."""
    return cfg.num_hidden_layers * 2.0 * 2.0 * cfg.q_dim * (new * before + new * (new + 1) / 2.0)


def run_57b(args) -> int:
    """The two workloads at the Qwen2-57B-A14B shape (see the module's docstring)."""
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors

    shape = SHAPE if args.workload == "mixed-small" else SHAPE_57B
    shape_name = "Qwen1.5-MoE-A2.7B shape" if args.workload == "mixed-small" else "Qwen2-57B-A14B shape"
    layers = args.layers or shape["num_hidden_layers"]
    raw = dict(shape)
    raw["num_hidden_layers"] = layers
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    peak = PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12
    mixed = args.workload in ("mixed", "mixed-small")
    context = {"mixed": 8192, "mixed-small": 4096, "long": 32768}[args.workload]
    log(f"drawing random weights on the device ({layers} layers, {args.dtype})")
    t0 = time.time()
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0").items()}
    gen = torch.Generator().manual_seed(1234)
    rnd = lambda n: torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist()
    base = {"metric": None, "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids"}
    sizes = {"layers": layers, "layers_of_shape": shape["num_hidden_layers"], "hidden": cfg.hidden_size,
             "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
             "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok, "moe_intermediate": cfg.moe_intermediate_size,
             "shared_intermediate": cfg.shared_expert_intermediate_size, "vocab": cfg.vocab_size, "page_size": PAGE}

    if mixed:
        n_dec, dec_ctx, n_pre, portion, pre_ctx = (32, 4096, 2, 512, 2048) if args.workload == "mixed" else \
            (8, 2048, 1, 64, 0)
        pages = (n_dec * context + n_pre * context) // PAGE
        runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=n_dec + n_pre,
                             max_seq_len=context, model=model)
        log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device")
        dec = [f"d{i}" for i in range(n_dec)]
        pre = [f"p{i}" for i in range(n_pre)]
        for r in dec + pre:  # the contexts the step starts from
            runner.add_request(r)
            for s in range(0, dec_ctx if r in dec else pre_ctx, 2048):
                runner.run_entries([(r, rnd(2048), [])])
        total = args.warmup + args.steps
        assert pre_ctx + total * portion <= context and dec_ctx + total <= context, f"fewer steps: the context is {context}"
        entries = lambda: [(r, rnd(1), [0]) for r in dec] + [(r, rnd(portion), []) for r in pre]
        for _ in range(args.warmup):
            runner.run_entries(entries())
        batches = [entries() for _ in range(args.steps)]
        torch.cuda.synchronize()
        t = time.perf_counter()
        for e in batches:
            runner.run_entries(e)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / args.steps
        tokens = n_dec + n_pre * portion
        mid = args.warmup + args.steps // 2
        cache_tokens = n_dec * (dec_ctx + mid) + n_pre * (pre_ctx + mid * portion)
        flops = linear_flops(cfg, tokens, n_dec) + n_dec * attention_flops(cfg, 1, dec_ctx + mid) \
            + n_pre * attention_flops(cfg, portion, pre_ctx + mid * portion)
        gbs = step_bytes(cfg, tokens, cache_tokens, elt) / dt / 1e9
        line = dict(base, metric=f"{shape_name}, mixed step ({n_dec} decodes at context {dec_ctx} beside {n_pre} prompt "
                                 f"portions of {portion}) through the step function, tokens/s",
                    value=round(tokens / dt, 1), ms_per_step=round(dt * 1e3, 3),
                    config=dict(sizes, model=shape_name, global_batch=n_dec + n_pre, seq_len=context,
                                tokens_per_step=tokens, parallelism="single GPU"),
                    prefill=None,
                    compute={"flops_per_step": flops, "frac": round(flops / dt / peak, 5)},
                    roofline={"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": round(gbs / PEAK_HBM_GBS, 5)}, points={})
        print(json.dumps(line), flush=True)
        return 0

    # ---- long context: batch 8, prompts of 16,384 to 32,000 tokens in portions of 2,048, then decoding ----
    batch, chunk = 8, 2048
    steps = args.steps
    lens = torch.randint(16384, 32001, (batch,), generator=gen).tolist()
    free, _ = torch.cuda.mem_get_info()
    per_page = cfg.num_hidden_layers * 2 * cfg.kv_dim * PAGE * elt
    pages = max(batch * context // PAGE, int(free * 0.85) // per_page)  # the pool fills what memory is left
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=batch, max_seq_len=context,
                         model=model)
    runner.capture_after = 1
    log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device, "
        f"{pages} pages ({pages * PAGE} tokens of cache)")
    engine = LLMEngine("", runner=runner, max_num_seqs=batch, max_model_len=context, max_num_batched_tokens=chunk)
    # (the first requests decode while the later prompts are still being read, about a hundred steps: room for those)
    slack = 8 * (32000 // chunk + 1) + 8
    params = SamplingParams(max_tokens=args.warmup + steps + slack, ignore_eos=True)
    assert max(lens) + args.warmup + steps + slack <= context, "fewer steps: the context is 32,768"
    ids = [engine.add_request(rnd(n), params) for n in lens]
    torch.cuda.synchronize()
    t = time.perf_counter()
    n_steps = 0
    while any(engine.scheduler.sequence(i).generated() == 0 for i in ids):
        engine.step()
        n_steps += 1
    torch.cuda.synchronize()
    t_pre = time.perf_counter() - t
    log(f"prompts of {lens}: {t_pre:.2f}s in {n_steps} steps")
    for _ in range(args.warmup):
        engine.step()
    torch.cuda.synchronize()
    before = engine.stats.tokens_out
    t = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t) / steps
    assert engine.stats.tokens_out - before == batch * steps, "a timed step was not a decode step of the whole batch"
    pre_flops = linear_flops(cfg, sum(lens), batch) + sum(attention_flops(cfg, n, 0) for n in lens)
    cache_tokens = sum(lens) + batch * (args.warmup + steps // 2 + batch)
    hit = experts_hit(engine.step, runner)
    gbs = step_bytes(cfg, batch, cache_tokens, elt, hit) / dt / 1e9
    line = dict(base, metric="Qwen2-57B-A14B shape, decode tok/s @ batch 8 after prompts of 16384-32000 tokens",
                value=round(batch / dt, 1), ms_per_step=round(dt * 1e3, 3),
                config=dict(sizes, model="Qwen2-57B-A14B shape", global_batch=batch, seq_len=context,
                            prompt_tokens=sum(lens), portion=chunk, cache_pages=pages, parallelism="single GPU"),
                prefill={"value": round(sum(lens) / t_pre, 1), "tokens": sum(lens), "ms": round(t_pre * 1e3, 1),
                         "frac": round(pre_flops / t_pre / peak, 5)},
                roofline={"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                          "frac": round(gbs / PEAK_HBM_GBS, 5),
                          "experts_hit_per_layer": round(hit, 1) if hit else None}, points={})
    print(json.dumps(line), flush=True)
    return 0


def run_portion(args) -> int:
    """One request's portion of --prefill-tokens tokens on top of --prefill-context tokens that it has read before
    (in portions of 2,048, untimed): the best of three, the logits of the last token only."""
    import torch
    from inferx_amd import ops
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.weights import random_tensors

    shape = SHAPE_57B if args.shape == "57b" else SHAPE
    shape_name = "Qwen2-57B-A14B shape" if args.shape == "57b" else "Qwen1.5-MoE-A2.7B shape"
    layers = args.layers or shape["num_hidden_layers"]
    raw = dict(shape, num_hidden_layers=layers, max_position_embeddings=65536)
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    ceilings = ops.measured_ceilings("cuda:0")
    log(f"drawing random weights on the device ({layers} layers, {args.dtype})")
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0").items()}
    n, before = args.prefill_tokens, args.prefill_context
    cap = -(-(n + before + PAGE) // PAGE) * PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=cap // PAGE, max_requests=1, max_seq_len=cap,
                         model=model)
    gen = torch.Generator().manual_seed(1234)
    rnd = lambda m: torch.randint(0, cfg.vocab_size, (m,), generator=gen).tolist()
    times = []
    for _ in range(3):
        runner.add_request("p")
        for at in range(0, before, PROMPT):
            runner.run_entries([("p", rnd(min(PROMPT, before - at)), [])])
        toks = rnd(n)
        torch.cuda.synchronize()
        t = time.perf_counter()
        runner.run_entries([("p", toks, [n - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t)
        runner.end_request("p")
    sec = min(times[1:])
    flops = linear_flops(cfg, n, 1) + attention_flops(cfg, n, before)
    peak = PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12
    line = {"metric": f"{shape_name}: prompt portion of {n} tokens on a context of {before}, tokens/s",
            "value": round(n / sec, 1), "unit": "tokens/s", "n_gpus": 1, "steps": 2, "warmup": 1,
            "ms_per_step": round(sec * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids",
            "config": {"model": shape_name, "global_batch": 1, "seq_len": n + before, "portion": n, "context": before,
                       "parallelism": "single GPU", "layers": layers, "layers_of_shape": shape["num_hidden_layers"],
                       "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                       "head_dim": cfg.head_dim, "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok,
                       "moe_intermediate": cfg.moe_intermediate_size,
                       "shared_intermediate": cfg.shared_expert_intermediate_size, "vocab": cfg.vocab_size,
                       "page_size": PAGE},
            "prefill": {"value": round(n / sec, 1), "tokens": n, "ms": round(sec * 1e3, 3),
                        "frac": round(flops / sec / peak, 5), "tflops": round(flops / sec / 1e12, 1)},
            "ceilings": ceilings}
    print(json.dumps(line), flush=True)
    return 0


def run_offline(args) -> int:
    """A finite batch of requests of mixed lengths through `LLMEngine.generate` (see the module's docstring)."""
    import random
    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors
    raw = dict(SHAPE)
    raw["num_hidden_layers"] = args.layers or SHAPE["num_hidden_layers"]
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    rnd = random.Random(0)
    n, live, budget, context = 96, 64, 4096, 4096
    lens = [rnd.choice([rnd.randint(5, 100), rnd.randint(100, 1000), rnd.randint(1000, 3000)]) for _ in range(n)]
    outs = [rnd.randint(4, 120) for _ in range(n)]
    gen = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, cfg.vocab_size, (m,), generator=gen).tolist() for m in lens]
    params = [SamplingParams(max_tokens=m, ignore_eos=True) for m in outs]
    log(f"drawing random weights on the device ({cfg.num_hidden_layers} layers, {args.dtype})")
    model = build_model(cfg.model_spec())
    weights = {k: rt.place(v) for k, v in random_tensors(model, 0, args.dtype, "cuda:0").items()}
    pages = 2200 if args.scarce else live * context // PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=live, max_seq_len=context,
                         model=model, max_step_tokens=budget)
    engine = LLMEngine("", runner=runner, max_num_seqs=live, max_model_len=context, max_num_batched_tokens=budget)
    engine.generate(prompts[:2], [SamplingParams(max_tokens=2, ignore_eos=True)] * 2)  # libraries' first calls
    steps0 = engine.stats.steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    got = engine.generate(prompts, params, with_reasons=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    bad = [(r, len(o), m) for (o, r), m in zip(got, outs) if r != "max_tokens" or len(o) != m]
    if bad:
        raise SystemExit(f"bench.py: {len(bad)} requests ended otherwise than asked, e.g. {bad[:3]}")
    runner.cache.check()
    total = sum(lens) + sum(outs)
    print(json.dumps({
        "metric": f"Qwen1.5-MoE-A2.7B offline batch, prompt + generated tokens/s ({n} requests, {live} at a time)",
        "value": round(total / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": engine.stats.steps - steps0,
        "warmup": 0, "ms_per_step": round(dt * 1e3 / max(engine.stats.steps - steps0, 1), 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random weights, token ids and lengths",
        "config": {"model": "Qwen1.5-MoE-A2.7B shape", "layers": cfg.num_hidden_layers,
                   "layers_of_shape": SHAPE["num_hidden_layers"], "requests": n, "max_num_seqs": live,
                   "max_num_batched_tokens": budget, "max_model_len": context, "pages": pages, "page_size": PAGE,
                   "parallelism": "single GPU"},
        "seconds": round(dt, 3), "prompt_tokens": sum(lens), "generated_tokens": sum(outs),
        "prompt_tokens_per_s": round(sum(lens) / dt, 1), "generated_tokens_per_s": round(sum(outs) / dt, 1),
        "preemptions": engine.stats.preemptions, "graphs_captured": len(runner._graphs)}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (32; 8 for mixed, 256 for long)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (4; 2 for mixed)")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the configuration has (sizes of a layer are never reduced)")
    ap.add_argument("--scarce", action="store_true", help="offline: so few pages that sequences are preempted")
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "mixed", "long", "mixed-small", "offline", "portion"],
                    help="decode, mixed-small: the Qwen1.5-MoE-A2.7B shape (decode is the default); mixed, long: the "
                         "Qwen2-57B-A14B shape")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT,
                    help="tokens of the prompt whose reading in one step is timed (2,048 is the contract's)")
    ap.add_argument("--prefill-context", type=int, default=0,
                    help="portion: tokens that the request has read before the timed portion")
    ap.add_argument("--shape", default="a27b", choices=["a27b", "57b"], help="portion: whose layer sizes")
    ap.add_argument("--prompt-len", type=int, default=PROMPT,
                    help="tokens of every request's prompt before it decodes (the context of the decode steps)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; --gpus N > 1 is not supported")
        return 2
    if args.steps is None:
        args.steps = {"decode": 32, "mixed": 8, "long": 256, "mixed-small": 24, "offline": 0, "portion": 2}[args.workload]
    if args.warmup is None:
        args.warmup = {"decode": 4, "mixed": 2, "long": 4, "mixed-small": 4, "offline": 0, "portion": 1}[args.workload]
    if args.workload == "offline":
        return run_offline(args)
    if args.workload == "portion":
        return run_portion(args)
    if args.workload != "decode":
        return run_57b(args)
    if args.layers is None:
        args.layers = SHAPE["num_hidden_layers"]

    import torch
    from inferx_amd.config import config_from_dict
    from inferx_amd.engine.engine import LLMEngine
    from inferx_amd.engine.runner import ModelRunner
    from inferx_amd.engine.runtime import Runtime
    from inferx_amd.parts import build_model
    from inferx_amd.sampling import SamplingParams
    from inferx_amd.weights import random_tensors

    raw = dict(SHAPE)
    raw["num_hidden_layers"] = args.layers
    cfg = config_from_dict(raw)
    rt = Runtime(args.dtype, "cuda:0")
    elt = 2 if args.dtype == "bfloat16" else 4
    from inferx_amd import ops
    ceilings = ops.measured_ceilings("cuda:0")  # before the weights take the memory
    log(f"measured on this machine: {ceilings}")
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    log(f"drawing random weights on the device ({args.layers} layers, {args.dtype})")
    t0 = time.time()
    model = build_model(cfg.model_spec())
    weights = random_tensors(model, seed=0, dtype=args.dtype, device="cuda:0")
    weights = {k: rt.place(v) for k, v in weights.items()}
    prompt_len = args.prompt_len
    # a request's prompt, the tokens it decodes while the later prompts are read (a step each portion), the steps
    reading = max_batch * -(-prompt_len // PROMPT)
    context_cap = max(CONTEXT, args.prefill_tokens, -(-(prompt_len + reading + 2 * args.steps + args.warmup + 3 * max_batch + 32) // PAGE) * PAGE)
    pages = max_batch * context_cap // PAGE
    runner = ModelRunner(cfg, weights, rt, page_size=PAGE, num_pages=pages, max_requests=max_batch,
                         max_seq_len=context_cap, model=model)
    runner.capture_after = 1  # a steady batch: its shape is captured at the first step, whatever --warmup says
    torch.cuda.synchronize()
    log(f"model ready in {time.time() - t0:.1f}s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB on the device")
    gen = torch.Generator().manual_seed(1234)

    def prompt(n=None):
        return torch.randint(0, cfg.vocab_size, (n or prompt_len,), generator=gen).tolist()

    def run_decode(batch, steps, warmup, single=0):
        """`batch` requests with prompts of `prompt_len` tokens through the engine (scheduler, step function, sampler):
        first their prompts, then `warmup` untimed and `steps` timed decode steps of the whole batch; then `single`
        more steps, each timed on its own (the device is waited for after every one of them, so they are a little
        slower than steps that follow each other).  Returns the time of the `steps` and the list of single times."""
        engine = LLMEngine("", runner=runner, max_num_seqs=batch, max_model_len=context_cap,
                           max_num_batched_tokens=max(PROMPT, batch))
        # (requests decode while the later prompts are still being read: room for those tokens too)
        params = SamplingParams(max_tokens=warmup + steps + single + batch * -(-prompt_len // PROMPT) + 3 * batch + 16,
                                ignore_eos=True)
        ids = [engine.add_request(prompt(), params) for _ in range(batch)]
        while any(engine.scheduler.sequence(i).generated() == 0 for i in ids):  # the prompts, one a step
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = engine.stats.tokens_out
        t = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert engine.stats.tokens_out - before == batch * steps, "a timed step was not a decode step of the whole batch"
        hit = experts_hit(engine.step, runner) if single else None
        singles = []
        for _ in range(single):
            t = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            singles.append(time.perf_counter() - t)
        for i in ids:
            engine.cancel(i)
        while engine.has_unfinished():
            engine.step()
        assert runner.cache.pools[0].used_pages == 0
        return dt, singles, hit

    # ---- prefill of one 2,048-token prompt ---------------------------------
    prefill = None
    if not args.no_prefill:
        log("prefill")
        n_pre = args.prefill_tokens
        times = []
        for i in range(3):
            runner.add_request("p")
            toks = prompt(n_pre)
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.run_entries([("p", toks, [n_pre - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            runner.end_request("p")
        sec = min(times[1:])
        flops = prefill_flops(cfg, n_pre)
        prefill = {"value": round(n_pre / sec, 1), "tokens": n_pre, "ms": round(sec * 1e3, 3),
                   "frac": round(flops / sec / (PEAK_TFLOPS["bf16" if elt == 2 else "fp32"] * 1e12), 5),
                   "tflops": round(flops / sec / 1e12, 1),
                   "frac_measured": round(flops / sec / (ceilings["mfma_bf16_tflops"] * 1e12), 5) if elt == 2 else None}
        log(f"prefill {prefill}")

    # ---- decode ----------------------------------------------------------------
    log(f"decode at batch {args.batch}")
    dt, singles, hit_per_layer = run_decode(args.batch, args.steps, args.warmup, single=args.steps)
    singles.sort()
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    context = prompt_len + args.warmup + args.steps // 2
    gbs = decode_bytes(cfg, args.batch, context, elt, hit_per_layer) / (dt / args.steps) / 1e9
    pts = {}
    for b in points:
        log(f"decode at batch {b}")
        steps = max(8, args.steps // 2)
        d, _, _ = run_decode(b, steps, max(2, args.warmup // 2))
        pts[f"decode_b{b}"] = round(b * steps / d, 1)

    line = {
        "metric": f"Qwen1.5-MoE-A2.7B decode tok/s @ batch {args.batch} ({prompt_len}-token prompts)",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 3),
        "step_ms": {"min": round(singles[0] * 1e3, 3), "median": round(singles[len(singles) // 2] * 1e3, 3)},
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if elt == 2 else "fp32", "data": "synthetic: seeded random weights and token ids",
        "config": {
            "model": "Qwen1.5-MoE-A2.7B shape", "global_batch": args.batch, "seq_len": context_cap, "prompt_len": prompt_len,
            "parallelism": "single GPU", "layers": args.layers, "layers_of_shape": SHAPE["num_hidden_layers"],
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "experts": cfg.num_experts, "top_k": cfg.num_experts_per_tok,
            "moe_intermediate": cfg.moe_intermediate_size, "shared_intermediate": cfg.shared_expert_intermediate_size,
            "vocab": cfg.vocab_size, "page_size": PAGE,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 5), "frac_measured": round(gbs / ceilings["hbm_read_gbs"], 5),
                     "experts_hit_per_layer": round(hit_per_layer, 1) if hit_per_layer else None},
        "ceilings": ceilings,
        "points": pts,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
