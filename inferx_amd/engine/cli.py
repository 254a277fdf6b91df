"""Command line: generate token ids for prompts given as token ids.

Option names and meanings are the reference server's where it has them
(src/support/options.cc:47-227: --model, --dtype, --max-num-seqs, --max-model-len,
--max-num-batched-tokens, --block-size, --num-gpu-blocks-override,
--kv-cache-memory-bytes, --gpu-memory-utilization, --enforce-eager, --device);
--dump-logits writes the file format of the reference's scripts/gen_reference_logits.py;
--log-level, --log-json, --log-file are the reference's (options.cc:218-227);
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


def _set_up_logging(level: str, as_json: bool, path: Optional[str]) -> None:
    """--log-level, --log-json, --log-file as the reference's server has them (src/support/options.cc:218-227)."""
    import logging

    class JsonLines(logging.Formatter):
        def format(self, record):
            return json.dumps({"time": round(record.created, 3), "level": record.levelname.lower(),
                               "logger": record.name, "message": record.getMessage()})

    handler = logging.FileHandler(path) if path else logging.StreamHandler(sys.stderr)
    handler.setFormatter(JsonLines() if as_json else logging.Formatter("%(levelname).1s %(name)s: %(message)s"))
    root = logging.getLogger("inferx_amd")
    root.handlers[:] = [handler]
    root.setLevel(getattr(logging, level.upper()))
    root.propagate = False


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="inferx-generate", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model_tag", nargs="?", help="checkpoint directory (positional form)")
    ap.add_argument("--model", help="checkpoint directory (config.json + model.safetensors)")
    ap.add_argument("--random-config", help="a config.json: make a folder of random weights from it and run that")
    ap.add_argument("--random-seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="auto", choices=["auto", "bfloat16", "bf16", "float", "float32", "fp32"],
                    help="auto and bfloat16 run the serving kernels; float32 runs everything in true 32-bit")
    ap.add_argument("--max-num-seqs", type=int, default=8, help="concurrent sequences")
    ap.add_argument("--max-model-len", type=int, default=2048, help="prompt + generation cap")
    ap.add_argument("--max-num-batched-tokens", type=int, default=None, help="token budget per scheduler step")
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-gpu-blocks-override", "--num-blocks", type=int, default=None,
                    help="cache pages (overrides sizing by memory)")
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
    ap.add_argument("--config", metavar="FILE", help="a TOML (.toml) or INI file of options by name; the command line wins")
    ap.add_argument("--log-level", default="warning", choices=["debug", "info", "warning", "error"],
                    help="what the engine reports on standard error (info: how the cache was sized; debug: every step)")
    ap.add_argument("--log-json", action="store_true", help="write the log as JSON lines")
    ap.add_argument("--log-file", help="append the log to a file instead of standard error")
    ap.add_argument("--dump-logits", metavar="FILE",
                    help="also write the float32 logits at every position of every prompt to FILE, one record per "
                         "prompt: 'IXRL', u32 version 1, u32 tokens, u32 vocab, i32 ids[tokens], f32 logits[tokens * vocab]")
    return ap


def _config_file_defaults(ap: argparse.ArgumentParser, path: str) -> dict:
    """Options from a TOML or INI file whose keys are the options' names (with dashes or underscores, without the
    leading ones); what the command line says wins.  (The reference's server takes such a file through --config,
    src/support/options.cc.)"""
    known = {a.dest: a for a in ap._actions if a.option_strings}
    try:
        with open(path, "rb") as f:
            raw = f.read()
        if path.endswith(".toml"):
            import tomli
            table = tomli.loads(raw.decode("utf-8"))
        else:
            import configparser
            cp = configparser.ConfigParser()
            cp.read_string("[options]\n" + raw.decode("utf-8") if not raw.lstrip().startswith(b"[") else raw.decode("utf-8"))
            table = {k: v for section in cp.sections() for k, v in cp.items(section)}
    except (OSError, ValueError, Exception) as e:  # noqa: B014  (any parser's complaint is a bad command line)
        ap.error(f"cannot read --config {path}: {e}")
    out = {}
    for key, value in table.items():
        dest = key.replace("-", "_")
        if dest not in known or dest == "config":
            ap.error(f"--config {path}: unknown option {key!r}")
        action = known[dest]
        if isinstance(action, argparse._StoreTrueAction):
            value = value if isinstance(value, bool) else str(value).strip().lower() in ("1", "true", "yes", "on")
        elif isinstance(action, argparse._AppendAction):
            value = [str(v) for v in (value if isinstance(value, list) else [value])]
        elif action.type is not None and not isinstance(value, bool):
            try:
                value = action.type(value)
            except (TypeError, ValueError):
                ap.error(f"--config {path}: {key} = {value!r} is not {action.type.__name__}")
        elif isinstance(value, (int, float)) and action.type is None:
            value = str(value)
        if action.choices and value not in action.choices:
            ap.error(f"--config {path}: {key} must be one of {', '.join(map(str, action.choices))}")
        out[dest] = value
    return out


def main(argv: Optional[List[str]] = None) -> int:
    ap = build_parser()
    first, _ = ap.parse_known_args(argv)
    if first.config:
        ap.set_defaults(**_config_file_defaults(ap, first.config))
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

    _set_up_logging(args.log_level, args.log_json, args.log_file)
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
            store = "float32" if args.dtype in ("float", "float32", "fp32") else "bfloat16"
            write_model_folder(cfg, args.random_seed, model, store)
        dtype = "float32" if args.dtype in ("float", "float32", "fp32") else "bfloat16"
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
