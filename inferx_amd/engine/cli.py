"""Command line: generate token ids for prompts given as token ids.

Option names and meanings are the reference server's where it has them
(src/support/options.cc:47-227: --model, --dtype, --max-num-seqs, --max-model-len,
--max-num-batched-tokens, --block-size, --num-gpu-blocks-override,
--kv-cache-memory-bytes, --gpu-memory-utilization, --enforce-eager, --device);
--dump-logits writes the file format of the reference's scripts/gen_reference_logits.py;
exit code 0 for --help and 2 for a bad command line (include/inferx/support/options.h:17-22).
There is no tokenizer and no server: prompts are token ids, output is one JSON
line per prompt.
"""
from __future__ import annotations

import argparse
import json
import struct
import sys
import tempfile
from typing import List, Optional


def _ids(text: str) -> List[int]:
    return [int(x) for x in text.replace(",", " ").split()]


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="inferx-generate", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model_tag", nargs="?", help="checkpoint directory (positional form)")
    ap.add_argument("--model", help="checkpoint directory (config.json + model.safetensors)")
    ap.add_argument("--random-config", help="a config.json: make a folder of random weights from it and run that")
    ap.add_argument("--random-seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="auto", choices=["auto", "bfloat16", "float", "float32"],
                    help="auto and bfloat16 run the serving kernels; float32 runs everything in true 32-bit")
    ap.add_argument("--max-num-seqs", type=int, default=8, help="concurrent sequences")
    ap.add_argument("--max-model-len", type=int, default=2048, help="prompt + generation cap")
    ap.add_argument("--max-num-batched-tokens", type=int, default=None, help="token budget per scheduler step")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-gpu-blocks-override", type=int, default=None, help="cache pages (overrides sizing by memory)")
    ap.add_argument("--kv-cache-memory-bytes", type=int, default=None, help="explicit cache budget in bytes")
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.92,
                    help="fraction of GPU memory the engine may use")
    ap.add_argument("--enforce-eager", action="store_true", help="no captured HIP graphs: every step launches its kernels one by one")
    ap.add_argument("--device", default="rocm", choices=["rocm", "cuda"], help="execution backend (one GPU)")
    ap.add_argument("--prompt-ids", action="append", default=[], help="a prompt as token ids, e.g. 1,2,3 (repeatable)")
    ap.add_argument("--prompt-file", help="file with one prompt of token ids per line")
    ap.add_argument("--max-tokens", type=int, default=16, help="generated tokens per prompt")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--min-p", type=float, default=0.0)
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("--repetition-penalty", type=float, default=1.0)
    ap.add_argument("--stop-token-ids", default="", help="comma-separated token ids that end a sequence")
    ap.add_argument("--min-tokens", type=int, default=0, help="stop tokens do not end a sequence before this many")
    ap.add_argument("--ignore-eos", action="store_true", help="generate through the model's end-of-sequence ids")
    ap.add_argument("--logprobs", type=int, default=None, metavar="N",
                    help="report each token's log-probability and those of the N most probable (0 to 20)")
    ap.add_argument("--seed", type=int, default=0, help="fixes the sampling draws")
    ap.add_argument("--dump-logits", metavar="FILE",
                    help="also write the float32 logits at every position of every prompt to FILE, one record per "
                         "prompt: 'IXRL', u32 version 1, u32 tokens, u32 vocab, i32 ids[tokens], f32 logits[tokens * vocab]")
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    ap = build_parser()
    args = ap.parse_args(argv)
    model = args.model or args.model_tag
    if (model is None) == (args.random_config is None):
        ap.error("give a model directory or --random-config FILE (one of them)")
    for name in ("max_num_seqs", "max_model_len", "block_size", "max_tokens"):
        if getattr(args, name) <= 0:
            ap.error(f"--{name.replace('_', '-')} must be positive")
    prompts = []
    try:
        prompts = [_ids(p) for p in args.prompt_ids]
        if args.prompt_file:
            with open(args.prompt_file) as f:
                prompts += [_ids(line) for line in f if line.strip()]
        stop = _ids(args.stop_token_ids)
    except (ValueError, OSError) as e:
        ap.error(f"cannot read the prompts: {e}")
    if not prompts or any(not p for p in prompts):
        ap.error("give at least one non-empty prompt (--prompt-ids or --prompt-file)")

    from ..config import ConfigError
    from ..sampling import SamplingParams
    from ..weights import CheckpointError
    from .engine import LLMEngine
    try:
        if args.random_config:
            from ..config import config_from_json
            from ..weights import write_model_folder
            with open(args.random_config) as f:
                cfg = config_from_json(f.read())
            model = tempfile.mkdtemp(prefix="inferx_random_")
            store = "float32" if args.dtype in ("float", "float32") else "bfloat16"
            write_model_folder(cfg, args.random_seed, model, store)
        dtype = "float32" if args.dtype in ("float", "float32") else "bfloat16"
        engine = LLMEngine(model, dtype, max_num_seqs=args.max_num_seqs, max_model_len=args.max_model_len,
                           max_num_batched_tokens=args.max_num_batched_tokens, block_size=args.block_size,
                           num_gpu_blocks_override=args.num_gpu_blocks_override,
                           kv_cache_memory_bytes=args.kv_cache_memory_bytes,
                           gpu_memory_utilization=args.gpu_memory_utilization, enforce_eager=args.enforce_eager)
        params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p,
                                top_k=args.top_k, min_p=args.min_p, presence_penalty=args.presence_penalty,
                                frequency_penalty=args.frequency_penalty,
                                repetition_penalty=args.repetition_penalty, stop_tokens=stop, seed=args.seed,
                                min_tokens=args.min_tokens, ignore_eos=args.ignore_eos,
                                want_logprobs=args.logprobs is not None, top_logprobs=args.logprobs or 0)
        if args.dump_logits:
            # the reference's logits file (scripts/gen_reference_logits.py:15-23), one record after the other
            with open(args.dump_logits, "wb") as f:
                for p in prompts:
                    logits = engine.prompt_logits(p).numpy().astype("<f4")
                    f.write(b"IXRL" + struct.pack("<III", 1, logits.shape[0], logits.shape[1]))
                    f.write(struct.pack(f"<{len(p)}i", *p))
                    f.write(logits.tobytes())
        results = engine.generate(prompts, params, with_reasons=True)
    except (ConfigError, CheckpointError, ValueError, OSError) as e:
        print(f"inferx-generate: {e}", file=sys.stderr)
        return 1
    for i, (tokens, reason) in enumerate(results):
        line = {"prompt": i, "output_token_ids": tokens, "finish_reason": reason}
        if args.logprobs is not None:
            line["logprobs"] = [{"logprob": chosen, "top": [[t, lp] for t, lp in top]}
                                for chosen, top in engine.last_completions[i].logprobs]
        print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
