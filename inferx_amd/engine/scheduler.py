"""The scheduler: all policy, no GPU.  It decides who runs, in which portions,
and what gives when pages run out; the model runner decides nothing.

Policies are the reference's (src/scheduler/scheduler.cc):
  admission   first come first served while fewer than `max_running` run; pages
              for the whole prompt are reserved; on a shortage the request stays
              at the head of the queue and admission stops (:294-370)
  budget      at most `max_batch_tokens` tokens a step; sequences with one
              pending token (decodes, last one-token portions) first, then
              prompts in running order take min(pending, budget) (:255-291)
  pages out   for a running sequence: the most recently admitted sequence is
              preempted (pages back, starts over with prompt + generated tokens,
              head of the queue); if the requester is the newest, the next
              newest yields; if it runs alone it finishes `out_of_memory`
              (:444-510, :206-229)
  context     a sequence that would pass `max_seq_len` finishes `context_limit`
  finishing   stop token (kept in the output), `max_tokens`, cancel (:677-758)
Pages go back the moment a sequence finishes or is preempted (:231-245).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Tuple

from ..cache.manager import (RESERVE_CONTEXT_FULL, RESERVE_OK, RESERVE_POOL_EMPTY, CacheManager)
from ..sampling.params import SamplingParams

FINISH_STOP, FINISH_LENGTH, FINISH_CANCELLED = "stop_token", "max_tokens", "cancelled"
FINISH_CONTEXT, FINISH_OOM = "context_limit", "out_of_memory"


@dataclass
class Sequence:
    rid: Hashable
    tokens: List[int]
    prompt_len: int
    params: SamplingParams
    cancelled: bool = False
    draws: int = 0  # sampled tokens so far: the counter of this request's random stream
    logprobs: List = field(default_factory=list)  # per generated token, when asked for

    def generated(self) -> int:
        return len(self.tokens) - self.prompt_len


@dataclass
class Completion:
    rid: Hashable
    output_tokens: List[int]
    reason: str
    logprobs: Optional[List] = None  # per output token (chosen log-probability, [(token, log-probability), ...])


@dataclass
class Contribution:
    rid: Hashable
    tokens: List[int]      # this step's tokens of the sequence
    first_position: int
    samples: bool          # the portion reaches the end of the sequence: its last row gives the next token


@dataclass
class StepPlan:
    contributions: List[Contribution] = field(default_factory=list)

    def entries(self):
        """(request, tokens, wanted places) for `build_step_batch`."""
        return [(c.rid, c.tokens, [len(c.tokens) - 1] if c.samples else []) for c in self.contributions]

    @property
    def num_tokens(self) -> int:
        return sum(len(c.tokens) for c in self.contributions)


class Scheduler:
    def __init__(self, cache: CacheManager, max_running: int = 8, max_batch_tokens: int = 2048,
                 max_seq_len: Optional[int] = None):
        if max_running <= 0 or max_batch_tokens <= 0:
            raise ValueError("max_running and max_batch_tokens must be positive")
        self.cache = cache
        self.max_running = min(max_running, cache.max_requests)
        self.max_batch_tokens = max_batch_tokens
        self.max_seq_len = min(max_seq_len or cache.max_seq_len, cache.max_seq_len)
        self.waiting: Deque[Sequence] = deque()
        self.running: List[Sequence] = []
        self.completed: List[Completion] = []
        self.preemptions = 0
        self._plan: Optional[StepPlan] = None

    # ---- requests --------------------------------------------------------
    def add_request(self, rid: Hashable, prompt: List[int], params: Optional[SamplingParams] = None) -> None:
        params = params or SamplingParams()
        params.validate()
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if any(s.rid == rid for s in list(self.waiting) + self.running):
            raise ValueError(f"request {rid!r} is already known")
        self.waiting.append(Sequence(rid, list(prompt), len(prompt), params))

    def cancel(self, rid: Hashable) -> None:
        for s in list(self.waiting) + self.running:
            if s.rid == rid:
                s.cancelled = True

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def take_completed(self) -> List[Completion]:
        out, self.completed = self.completed, []
        return out

    def sequence(self, rid) -> Sequence:
        for s in self.running:
            if s.rid == rid:
                return s
        raise KeyError(rid)

    # ---- internals ---------------------------------------------------------
    def _pending(self, s: Sequence) -> int:
        return len(s.tokens) - self.cache.cached(s.rid)

    def _retire(self, s: Sequence, reason: str) -> None:
        self.completed.append(Completion(s.rid, s.tokens[s.prompt_len:], reason,
                                         list(s.logprobs) if s.logprobs else None))
        if s.rid in self.cache:
            self.cache.free(s.rid)

    def _preempt(self, index: int) -> None:
        victim = self.running.pop(index)
        self.cache.free(victim.rid)
        self.waiting.appendleft(victim)
        self.preemptions += 1

    def _admit(self) -> None:
        while self.waiting and len(self.running) < self.max_running:
            s = self.waiting[0]
            if s.cancelled:
                self.waiting.popleft()
                self._retire(s, FINISH_CANCELLED)
                continue
            if len(s.tokens) > self.max_seq_len:
                self.waiting.popleft()
                self._retire(s, FINISH_OOM)
                continue
            if not self.cache.can_add():
                return
            self.cache.add(s.rid)
            if self.cache.reserve(s.rid, len(s.tokens)) != RESERVE_OK:
                self.cache.free(s.rid)  # not a preemption site: it waits at the head of the queue
                return
            self.waiting.popleft()
            self.running.append(s)

    def _take(self) -> List[int]:
        take = [0] * len(self.running)
        budget = self.max_batch_tokens
        for i, s in enumerate(self.running):
            if budget > 0 and self._pending(s) == 1:
                take[i] = 1
                budget -= 1
        for i, s in enumerate(self.running):
            pending = self._pending(s)
            if budget > 0 and pending > 1:
                take[i] = min(pending, budget)
                budget -= take[i]
        return take

    # ---- one step ------------------------------------------------------------
    def prepare_step(self) -> Optional[StepPlan]:
        """Decide the next step.  None when nothing can run."""
        if self._plan is not None:
            raise RuntimeError("prepare_step called twice without commit_step")
        for s in [s for s in self.running if s.cancelled]:
            self.running.remove(s)
            self._retire(s, FINISH_CANCELLED)
        self._admit()
        take: List[int] = []
        for _ in range(len(self.running) + 1):
            if not self.running:
                return None
            take = self._take()
            replan = False
            for i, s in enumerate(self.running):
                if take[i] == 0:
                    continue
                status = self.cache.reserve(s.rid, self.cache.cached(s.rid) + take[i])
                if status == RESERVE_OK:
                    continue
                if status == RESERVE_CONTEXT_FULL:
                    self.running.pop(i)
                    self._retire(s, FINISH_CONTEXT)
                else:
                    victim = len(self.running) - 1
                    if victim == i:
                        if len(self.running) == 1:
                            self.running.pop(i)
                            self._retire(s, FINISH_OOM)
                            replan = True
                            break
                        victim = len(self.running) - 2
                    self._preempt(victim)
                replan = True
                break
            if not replan:
                break
        if not self.running:
            return None
        plan = StepPlan()
        for i, s in enumerate(self.running):
            if take[i] == 0:
                continue
            at = self.cache.cached(s.rid)
            plan.contributions.append(Contribution(s.rid, s.tokens[at:at + take[i]], at,
                                                   samples=at + take[i] == len(s.tokens)))
        if not plan.contributions:
            return None
        self._plan = plan
        return plan

    def commit_step(self, sampled: List[int], logprobs: Optional[List] = None) -> None:
        """`sampled`: one token per contribution that samples, in order; `logprobs`: what the sampler reported
        for those rows (or None)."""
        plan, self._plan = self._plan, None
        if plan is None:
            raise RuntimeError("commit_step without prepare_step")
        want = sum(1 for c in plan.contributions if c.samples)
        if len(sampled) != want:
            raise ValueError(f"{len(sampled)} sampled tokens for {want} sampling rows")
        it = iter(sampled)
        lp_it = iter(logprobs) if logprobs is not None else None
        finished: List[Tuple[Sequence, str]] = []
        by_id = {s.rid: s for s in self.running}
        for c in plan.contributions:
            s = by_id[c.rid]
            self.cache.commit(c.rid, len(c.tokens))
            if not c.samples:
                continue
            token = int(next(it))
            lp = next(lp_it) if lp_it is not None else None
            if lp is not None:
                s.logprobs.append(lp)
            s.tokens.append(token)
            s.draws += 1
            if token in s.params.stop_tokens and s.generated() > s.params.min_tokens:
                finished.append((s, FINISH_STOP))
            elif s.generated() >= s.params.max_tokens:
                finished.append((s, FINISH_LENGTH))
        for s, reason in finished:
            self.running.remove(s)
            self._retire(s, reason)
