"""The engine: model runner + scheduler + sampler in one loop, and the Python
entry point.

    engine = LLMEngine("model_dir", dtype="bfloat16")
    outputs = engine.generate([[1, 2, 3], [4, 5]], SamplingParams(max_tokens=8))

One iteration is prepare_step -> step -> sample -> commit_step (reference:
Engine::Impl::RunModel, src/engine/engine.cc:526-666).  Option names follow the
reference's command line (src/support/options.cc:47-174).  Token ids in, token
ids out: tokenizers and servers are not part of this engine.
"""
from __future__ import annotations

import dataclasses
import logging
import time
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Union

import torch

from ..config import config_from_directory
from ..parts import build_model
from ..sampling import Sampler, SamplingParams
from ..weights import load_weights
from .batch import build_step_batch
from .runner import ModelRunner
from .runtime import Runtime
from .scheduler import Completion, Scheduler

KV_HEADROOM_BYTES = 1 << 30
log = logging.getLogger("inferx_amd.engine")


def resolve_kv_blocks(block_bytes: int, *, explicit_blocks: Optional[int] = None,
                      kv_cache_memory_bytes: Optional[int] = None, gpu_memory_utilization: float = 0.92,
                      total_bytes: int = 0, used_bytes: int = 0, min_blocks: int = 1,
                      headroom_bytes: int = KV_HEADROOM_BYTES) -> int:
    """How many pages the pool gets.  An explicit count wins, unchecked; else explicit bytes; else
    utilization * total - used - headroom.  Fewer than `min_blocks` (one sequence of the longest length) is an
    error that says which option to change (reference: ResolveKvBlocks, src/engine/kv_autosize.cc:10-47;
    vectors tests/unit/kv_autosize_test.cc:14-78)."""
    if explicit_blocks is not None:
        if explicit_blocks <= 0:
            raise ValueError("--num-gpu-blocks-override must be positive")
        return explicit_blocks
    if block_bytes <= 0:
        raise ValueError(f"sizing the cache needs a positive page size in bytes, got {block_bytes}")
    if kv_cache_memory_bytes is not None:
        blocks = kv_cache_memory_bytes // block_bytes
        if blocks < min_blocks:
            raise ValueError(f"--kv-cache-memory-bytes {kv_cache_memory_bytes} holds only {blocks} pages of "
                             f"{block_bytes} bytes but one sequence of --max-model-len needs {min_blocks}; raise "
                             "the budget or lower --max-model-len")
        return blocks
    if not 0.0 < gpu_memory_utilization <= 1.0:
        raise ValueError("--gpu-memory-utilization must be within (0, 1]")
    budget = int(gpu_memory_utilization * total_bytes) - used_bytes - headroom_bytes
    blocks = max(0, budget) // block_bytes
    if blocks < min_blocks:
        raise ValueError(f"the cache does not fit: --gpu-memory-utilization {gpu_memory_utilization} of "
                         f"{total_bytes} bytes leaves {max(budget, 0)} bytes after the {used_bytes} already in use "
                         f"(weights, activations) and {headroom_bytes} of headroom, which holds {blocks} pages of "
                         f"{block_bytes} bytes but one sequence of --max-model-len needs {min_blocks}; raise "
                         "--gpu-memory-utilization or lower --max-model-len")
    return blocks


@dataclass
class Stats:
    steps: int = 0
    tokens_in: int = 0
    tokens_out: int = 0
    preemptions: int = 0
    step_seconds: float = 0.0


PROMPT_LOGITS_ROWS = 512  # rows per step of `LLMEngine.prompt_logits`


class LLMEngine:
    def __init__(self, model: str, dtype: str = "bfloat16", *, max_num_seqs: int = 8, max_model_len: int = 2048,
                 max_num_batched_tokens: Optional[int] = None, block_size: int = 16,
                 num_gpu_blocks_override: Optional[int] = None, kv_cache_memory_bytes: Optional[int] = None,
                 gpu_memory_utilization: float = 0.92, device: str = "cuda:0", enforce_eager: bool = False,
                 runner: Optional[ModelRunner] = None):
        if max_num_batched_tokens is None:
            max_num_batched_tokens = max(2048, max_model_len)  # reference: options.cc:332-336
        if runner is None:
            config = config_from_directory(model)
            rt = Runtime(dtype, device)
            net = build_model(config.model_spec())
            weights = load_weights(net, model, rt)
            # page count needs the per-token bytes, which need the cache plan: lay out with one page, then size
            probe = ModelRunner(config, weights, rt, page_size=block_size, num_pages=1, max_requests=max_num_seqs,
                                max_seq_len=max_model_len, model=net, use_graphs=not enforce_eager,
                                max_step_tokens=max_num_batched_tokens)
            block_bytes = probe.kv_bytes_per_token() * block_size
            torch.cuda.empty_cache()  # what loading and restacking the weights left cached is free for the pages
            free, total = torch.cuda.mem_get_info(rt.device)
            pages = resolve_kv_blocks(max(block_bytes, 1), explicit_blocks=num_gpu_blocks_override,
                                      kv_cache_memory_bytes=kv_cache_memory_bytes,
                                      gpu_memory_utilization=gpu_memory_utilization, total_bytes=total,
                                      used_bytes=total - free, min_blocks=-(-max_model_len // block_size))
            if num_gpu_blocks_override is None:
                # Windowed groups take no more than window + step per request, whatever the page count: what they
                # leave of the budget goes to the groups that keep every token.
                growing = sum(probe.page_bytes(g) for g, n in enumerate(probe.group_needs)
                              if probe.pages_of_group(n, pages + 1) > probe.pages_of_group(n, pages))
                if growing:
                    pages += max(0, pages * block_bytes - probe.cache_bytes(pages)) // growing
            pages = min(pages, max_num_seqs * -(-max_model_len // block_size))  # more could never be used
            # (the reference logs the same figures: AutosizeKvBlocksOnDevice, src/engine/kv_autosize.cc:65-71)
            log.info("cache: %d bytes on the device, %d already in use, utilization %s, page %d bytes -> %d pages of "
                     "%d tokens (%d bytes) in %d group(s)", total, total - free, gpu_memory_utilization, block_bytes,
                     pages, block_size, probe.cache_bytes(pages), len(probe.group_needs))
            probe._lay_out_cache(pages)
            runner = probe
        self.runner = runner
        self.scheduler = Scheduler(runner.cache, max_running=max_num_seqs, max_batch_tokens=max_num_batched_tokens,
                                   max_seq_len=max_model_len)
        self.sampler = Sampler(runner.rt)
        self.stats = Stats()
        self._next_id = 0
        self.plan_ahead = True  # plan and lay out the next step while the device runs this one
        self._ahead = None      # (plan, batch) made that way
        self._failed: Optional[str] = None  # set when a launched step could not be finished

    # ---- requests -----------------------------------------------------------
    def add_request(self, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    request_id: Optional[Hashable] = None) -> Hashable:
        vocab = self.runner.spec.vocab_size
        bad = [t for t in prompt_token_ids if not 0 <= int(t) < vocab]
        if bad:
            raise ValueError(f"prompt token id {bad[0]} is outside the vocabulary of {vocab}")
        if request_id is None:
            request_id = self._next_id
            self._next_id += 1
        # the model's end-of-sequence ids join the request's stop tokens unless it asks to generate through them
        # (reference: src/engine/engine.cc:819-823)
        params = params or SamplingParams()
        eos = [t for t in getattr(self.runner.config, "eos_token_ids", []) if t not in params.stop_tokens]
        if eos and not params.ignore_eos:
            params = dataclasses.replace(params, stop_tokens=list(params.stop_tokens) + eos)
        self.scheduler.add_request(request_id, [int(t) for t in prompt_token_ids], params)
        return request_id

    def cancel(self, request_id: Hashable) -> None:
        self.scheduler.cancel(request_id)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work()

    # ---- the loop -------------------------------------------------------------
    def step(self) -> List[Completion]:
        """One scheduler step.  Returns the requests that finished in it.

        While the device runs the step, the host already plans and lays out the next one (the scheduler takes a
        step in two halves: `launched` and `resolve`); when the sampled tokens arrive they are written into that
        layout, which is then ready to go.  If one of its sequences has just ended the plan is dropped and made
        again at the next call."""
        if self._failed is not None:
            raise RuntimeError(f"the engine stopped after an error inside a running step: {self._failed}")
        ahead, self._ahead = self._ahead, None
        try:
            if ahead is not None:
                plan, batch = ahead
            else:
                plan = self.scheduler.prepare_step()
                if plan is None:
                    return self.scheduler.take_completed()
                batch = build_step_batch(self.runner.cache, plan.entries())
            t0 = time.perf_counter()
            rows = [self.scheduler.sequence(c.rid).sampling_row() for c in plan.contributions if c.samples]
        except BaseException:
            # nothing of this step counts: the plan is dropped (its pages stay reserved for the sequences) and the
            # next call plans afresh, so a bad request can be cancelled and the others go on
            self.scheduler.abandon_step()
            raise
        stateful = self.runner.keeps_state
        try:
            logits = self.runner.step(batch)
            pending = self.sampler.launch(logits, rows)
        except BaseException as e:
            self.scheduler.abandon_step()
            if stateful:
                # Pages would be rewritten with the same values when the step is planned again; what parts keep per
                # request (state slots) may have been advanced by the failed step and would be advanced twice.
                self._failed = f"{type(e).__name__}: {e} (a model with per-request state cannot run a step again)"
            raise
        self.scheduler.launched()
        try:
            return self._finish_step(plan, pending, t0)
        except BaseException as e:
            self._failed = f"{type(e).__name__}: {e}"
            raise

    def _finish_step(self, plan, pending, t0) -> List[Completion]:
        nxt = nbatch = None
        if self.plan_ahead:
            nxt = self.scheduler.prepare_step()
            if nxt is not None:
                nbatch = build_step_batch(self.runner.cache, nxt.entries())
        sampled = pending.result()
        dropped = self.scheduler.resolve(sampled, self.sampler.last_logprobs)
        if nxt is not None and not dropped:
            nbatch.token_ids[:] = self.scheduler.plan_token_values(nxt)
            self._ahead = (nxt, nbatch)
        self.stats.steps += 1
        self.stats.tokens_in += plan.num_tokens
        self.stats.tokens_out += len(sampled)
        self.stats.preemptions = self.scheduler.preemptions
        self.stats.step_seconds += time.perf_counter() - t0
        done = self.scheduler.take_completed()
        if log.isEnabledFor(logging.DEBUG):
            log.debug("step %d: %d tokens of %d requests in, %d sampled, %d finished, %.3f ms", self.stats.steps,
                      plan.num_tokens, len(plan.contributions), len(sampled), len(done),
                      (time.perf_counter() - t0) * 1e3)
        return done

    def prompt_logits(self, prompt_token_ids: Sequence[int]) -> torch.Tensor:
        """float32 logits [len(prompt), vocab] (on the CPU) at every position of a prompt, run through the step
        function in portions under the token budget, as a request of its own that holds pages only meanwhile
        (what the reference's scripts/gen_reference_logits.py:15-23 writes for its own model).  Not to be called
        while requests are in flight."""
        if self.scheduler.has_work():
            raise RuntimeError("prompt_logits runs beside no other request")
        ids = [int(t) for t in prompt_token_ids]
        vocab = self.runner.spec.vocab_size
        if not ids or any(not 0 <= t < vocab for t in ids):
            raise ValueError("prompt_logits needs a non-empty prompt of token ids inside the vocabulary")
        rid = ("prompt_logits", self._next_id)
        self._next_id += 1
        self.runner.add_request(rid)
        rows = []
        try:
            # every row is wanted, so a portion's logits are portion x vocabulary floats beside the cache: portions
            # of at most PROMPT_LOGITS_ROWS whatever the scheduler's budget (512 x 152k x 4 bytes = 0.3 GB)
            budget = min(self.scheduler.max_batch_tokens, PROMPT_LOGITS_ROWS)
            for at in range(0, len(ids), budget):
                part = ids[at:at + budget]
                rows.append(self.runner.run_entries([(rid, part, list(range(len(part))))]).cpu())
        finally:
            self.runner.end_request(rid)
        return torch.cat(rows)

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 with_reasons: bool = False):
        """Generated token ids per prompt, in the order of the prompts."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt is needed")
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, params)]
        done: Dict[Hashable, Completion] = {}
        while len(done) < len(ids):
            before = self.stats.steps
            finished = self.step()
            for c in finished:
                done[c.rid] = c
            if not finished and self.stats.steps == before:
                # no step ran and nobody finished: nothing would change by asking again
                if self.scheduler.has_work():
                    raise RuntimeError("the scheduler has requests but can neither run nor end any of them")
                break
        missing = [i for i in ids if i not in done]
        if missing:
            raise RuntimeError(f"requests {missing} never finished")
        self.last_completions = [done[i] for i in ids]  # with finish reasons and log-probabilities
        if with_reasons:
            return [(done[i].output_tokens, done[i].reason) for i in ids]
        return [done[i].output_tokens for i in ids]
