"""The scheduler: all policy, no GPU.  It decides who runs, in which portions,
and what gives when pages run out; the model runner decides nothing.  The
decisions are made in the host library (inferx_amd/csrc/host/scheduler.cc); this
module is its face and keeps what only Python has use for (sampling
parameters, log-probabilities).

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

import ctypes
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional

import numpy as np

from ..cache.manager import CacheManager, host_lib
from ..sampling.params import SamplingParams

FINISH_STOP, FINISH_LENGTH, FINISH_CANCELLED = "stop_token", "max_tokens", "cancelled"
FINISH_CONTEXT, FINISH_OOM = "context_limit", "out_of_memory"
_REASONS = [FINISH_STOP, FINISH_LENGTH, FINISH_CANCELLED, FINISH_CONTEXT, FINISH_OOM]  # the library's numbering


class GeneratedTokens:
    """The tokens a sequence has generated so far: its length is known at once, the tokens are fetched from the
    library only when somebody iterates (penalties)."""

    def __init__(self, sched: "Scheduler", ident: int, prompt_len: int, count: int):
        self._sched, self._ident, self._prompt_len, self._count = sched, ident, prompt_len, count

    def __len__(self) -> int:
        return self._count

    def __iter__(self):
        return iter(self._sched._tokens(self._ident, self._prompt_len, self._count))


class Sequence:
    """A look at one request the scheduler knows."""

    def __init__(self, sched: "Scheduler", rid: Hashable):
        self._sched, self.rid = sched, rid
        self._ident = sched.cache.intern(rid)
        self.params: SamplingParams = sched._params[rid]

    def _info(self):
        p, n, d = ctypes.c_int32(), ctypes.c_int64(), ctypes.c_int64()
        if self._sched._lib.ixh_sched_seq_info(self._sched._h, self._ident, ctypes.byref(p), ctypes.byref(n),
                                               ctypes.byref(d)) != 0:
            raise KeyError(self.rid)
        return p.value, n.value, d.value

    @property
    def prompt_len(self) -> int:
        return self._info()[0]

    @property
    def draws(self) -> int:
        """Sampled tokens so far: the counter of this request's random stream."""
        return self._info()[2]

    @property
    def tokens(self) -> List[int]:
        return self._sched._tokens(self._ident, 0, self._info()[1])

    def generated(self) -> int:
        p, n, _ = self._info()
        return n - p

    def sampling_row(self):
        """(parameters, draws so far, generated tokens) as the sampler wants them."""
        p, n, d = self._info()
        return self.params, d, GeneratedTokens(self._sched, self._ident, p, n - p)


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


def _p32(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


def _p64(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))


class Scheduler:
    def __init__(self, cache: CacheManager, max_running: int = 8, max_batch_tokens: int = 2048,
                 max_seq_len: Optional[int] = None):
        if max_running <= 0 or max_batch_tokens <= 0:
            raise ValueError("max_running and max_batch_tokens must be positive")
        self.cache = cache
        self.max_running = min(max_running, cache.max_requests)
        self.max_batch_tokens = max_batch_tokens
        self.max_seq_len = min(max_seq_len or cache.max_seq_len, cache.max_seq_len)
        if cache.max_step_tokens is not None and max_batch_tokens > cache.max_step_tokens:
            raise ValueError(f"the cache was made for steps of at most {cache.max_step_tokens} tokens of a request, "
                             f"the token budget is {max_batch_tokens}")
        self._lib = host_lib()
        self._h = self._lib.ixh_sched_create(cache._h, self.max_running, self.max_batch_tokens, self.max_seq_len)
        if not self._h:
            raise RuntimeError("the scheduler could not be created")
        self._params: Dict[Hashable, SamplingParams] = {}
        self._logprobs: Dict[Hashable, List] = {}
        self._in_flight: Optional[List[Hashable]] = None
        self._plan: Optional[StepPlan] = None

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ixh_sched_destroy(self._h)
            self._h = None

    def _error(self) -> str:
        return self._lib.ixh_sched_error(self._h).decode("utf-8", "replace")

    def _tokens(self, ident: int, start: int, count: int) -> List[int]:
        buf = np.empty(max(count, 1), np.int32)
        n = self._lib.ixh_sched_seq_tokens(self._h, ident, start, _p32(buf), count)
        return buf[:max(n, 0)].tolist()

    # ---- requests --------------------------------------------------------
    def add_request(self, rid: Hashable, prompt: List[int], params: Optional[SamplingParams] = None) -> None:
        params = params or SamplingParams()
        params.validate()
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if rid in self._params:
            raise ValueError(f"request {rid!r} is already known")
        ids = np.asarray(prompt, dtype=np.int32)
        stop = np.asarray(sorted(params.stop_tokens), dtype=np.int32)
        rc = self._lib.ixh_sched_add(self._h, self.cache.intern(rid), _p32(ids), len(ids), int(params.max_tokens),
                                     int(params.min_tokens), _p32(stop) if len(stop) else None, len(stop))
        if rc != 0:
            self.cache.forget(rid)
            raise ValueError(f"request {rid!r} was refused by the scheduler ({rc})")
        self._params[rid] = params
        self._logprobs[rid] = []

    def cancel(self, rid: Hashable) -> None:
        if rid in self._params:
            self._lib.ixh_sched_cancel(self._h, self.cache.intern(rid))

    def has_work(self) -> bool:
        return bool(self._lib.ixh_sched_has_work(self._h))

    @property
    def preemptions(self) -> int:
        return self._lib.ixh_sched_preemptions(self._h)

    def _list(self, which: int) -> List[Sequence]:
        n = self._lib.ixh_sched_list(self._h, which, None, 0)
        buf = np.empty(max(n, 1), np.int64)
        self._lib.ixh_sched_list(self._h, which, _p64(buf), n)
        return [Sequence(self, self.cache.name_of(int(i))) for i in buf[:n]]

    @property
    def running(self) -> List[Sequence]:
        """The running sequences in order of admission."""
        return self._list(0)

    @property
    def waiting(self) -> List[Sequence]:
        """The waiting sequences from the head of the queue."""
        return self._list(1)

    def sequence(self, rid) -> Sequence:
        if rid not in self._params:
            raise KeyError(rid)
        return Sequence(self, rid)

    def take_completed(self) -> List[Completion]:
        n = self._lib.ixh_sched_num_completed(self._h)
        out = []
        for i in range(n):
            ident, reason, count = ctypes.c_int64(), ctypes.c_int32(), ctypes.c_int32()
            self._lib.ixh_sched_completed(self._h, i, ctypes.byref(ident), ctypes.byref(reason), ctypes.byref(count))
            buf = np.empty(max(count.value, 1), np.int32)
            self._lib.ixh_sched_completed_tokens(self._h, i, _p32(buf))
            rid = self.cache.name_of(ident.value)
            lps = self._logprobs.pop(rid, None)
            self._params.pop(rid, None)
            out.append(Completion(rid, buf[:count.value].tolist(), _REASONS[reason.value], list(lps) if lps else None))
            self.cache.forget(rid)
        if n:
            self._lib.ixh_sched_clear_completed(self._h)
        return out

    # ---- one step ------------------------------------------------------------
    def prepare_step(self) -> Optional[StepPlan]:
        """Decide the next step.  None when nothing can run."""
        n = self._lib.ixh_sched_prepare(self._h)
        if n < 0:
            raise RuntimeError(self._error())
        if n == 0:
            return None
        total = self._lib.ixh_sched_plan_tokens(self._h)
        rids, first = np.empty(n, np.int64), np.empty(n, np.int64)
        counts, samples, tokens = np.empty(n, np.int32), np.empty(n, np.int32), np.empty(total, np.int32)
        self._lib.ixh_sched_plan(self._h, _p64(rids), _p64(first), _p32(counts), _p32(samples), _p32(tokens))
        plan, at, flat = StepPlan(), 0, tokens.tolist()
        for i in range(n):
            c = int(counts[i])
            plan.contributions.append(Contribution(self.cache.name_of(int(rids[i])), flat[at:at + c], int(first[i]),
                                                   bool(samples[i])))
            at += c
        self._plan = plan
        return plan

    def abandon_step(self) -> None:
        """The planned step will not run (its launch failed): drop the plan; the next `prepare_step` plans afresh."""
        self._lib.ixh_sched_abandon(self._h)
        self._plan = None

    def commit_step(self, sampled: List[int], logprobs: Optional[List] = None) -> None:
        """`sampled`: one token per contribution that samples, in order; `logprobs`: what the sampler reported
        for those rows (or None).  `launched` and `resolve` in one."""
        plan = self._plan
        if plan is None:
            raise RuntimeError("commit_step without prepare_step")
        want = sum(1 for c in plan.contributions if c.samples)
        if len(sampled) != want:
            raise ValueError(f"{len(sampled)} sampled tokens for {want} sampling rows")
        self.launched()
        self.resolve(sampled, logprobs)

    # ---- a step in two halves: the next one can be planned while this one runs -----------------
    def launched(self) -> None:
        """The planned step has been handed to the device.  Its tokens count as cached from now on, and every
        sequence that samples holds a place for the value that is on its way; `prepare_step` may be called
        before `resolve` brings the values (the new plan's tokens of such places read -1 until then)."""
        plan, self._plan = self._plan, None
        if plan is None:
            raise RuntimeError("launched without prepare_step")
        rc = self._lib.ixh_sched_launched(self._h)
        if rc < 0:
            self._plan = plan
            raise RuntimeError(self._error())
        self._in_flight = [c.rid for c in plan.contributions if c.samples]

    def resolve(self, sampled: List[int], logprobs: Optional[List] = None) -> bool:
        """The sampled values of the launched step.  True if a step planned meanwhile was dropped because one of
        its sequences has just ended: plan again."""
        rows, self._in_flight = self._in_flight, None
        if rows is None:
            raise RuntimeError("resolve without a launched step")
        arr = np.asarray([int(t) for t in sampled], dtype=np.int32)
        rc = self._lib.ixh_sched_resolve(self._h, _p32(arr) if len(arr) else None, len(arr))
        if rc == -2:
            self._in_flight = rows
            raise ValueError(self._error())
        if rc < 0:
            raise RuntimeError(self._error())
        if logprobs is not None:
            for rid, lp in zip(rows, logprobs):
                if lp is not None and rid in self._logprobs:
                    self._logprobs[rid].append(lp)
        if rc == 1:
            self._plan = None
        return rc == 1

    def plan_token_values(self, plan: StepPlan) -> np.ndarray:
        """The tokens of the planned step, flat in the order of its contributions, as they are now (after `resolve`
        no place is open any more); the plan's contributions are brought up to date too."""
        if self._plan is not plan or not self._lib.ixh_sched_is_planned(self._h):
            raise RuntimeError("this plan is not the planned step")
        tokens = np.empty(plan.num_tokens, np.int32)
        self._lib.ixh_sched_plan_token_values(self._h, _p32(tokens))
        at, flat = 0, tokens.tolist()
        for c in plan.contributions:
            n = len(c.tokens)
            c.tokens = flat[at:at + n]
            at += n
        return tokens
