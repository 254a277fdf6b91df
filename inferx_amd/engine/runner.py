"""The step function and the memory it runs on.

`ModelRunner` owns the model (parts with their weights bound), the cache
memory (pages of keys and values per group, state slots) and the host-side
`CacheManager`.  `step(batch)` runs exactly the tokens the batch brings, as one
batch, against the cache that earlier steps left, and returns float32 logits
at the wanted rows (reference: Qwen2Model::Step, src/model/qwen2.cc:2246-2277;
PrepareBatchInputs :564-817).  It holds no policy: who runs, in which portions,
and what happens when pages run out is decided above it (scheduler, replay).

Steps in which every request brings one token are launch-bound, so they are
captured once per (batch size, context bucket) into a HIP graph and replayed
(reference: CaptureDecodeGraph, src/model/qwen2.cc:1588-1712).  The graph reads
its indices from one static device buffer that each step refills with a single
copy; kernels, buffers and results are those of the eager path.
"""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, GroupLayout, pages_for_window
from ..config import config_from_directory
from ..parts import build_model
from ..weights import load_weights
from .batch import Entry, StepBatch, build_step_batch
from .runtime import CacheBinding, Runtime, StepContext

# what a block of per-request state may be made of
STATE_TYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32, "int64": torch.int64}
N_FIXED = 7  # token_ids, positions, seq_of_token, q_start, seq_lens, state_slots, logits_rows


def _pack(batch: StepBatch, out: Optional[np.ndarray] = None) -> Tuple[List[int], np.ndarray]:
    """The batch's arrays one after the other as int32; into `out` if it is given and has their size."""
    parts = [batch.token_ids, batch.positions, batch.seq_of_token, batch.q_start, batch.seq_lens,
             batch.state_slots, batch.logits_rows] + list(batch.slots) + [t.reshape(-1) for t in batch.block_tables]
    sizes = [int(p.size) for p in parts]
    if not sum(sizes):
        return sizes, np.zeros(0, np.int32)
    flat = [np.ascontiguousarray(p, dtype=np.int32).reshape(-1) for p in parts]
    if out is not None and out.size == sum(sizes):
        return sizes, np.concatenate(flat, out=out)
    return sizes, np.concatenate(flat)


class ModelRunner:
    def __init__(self, config, weights: Dict[str, torch.Tensor], rt: Runtime, *, page_size: int = 16,
                 num_pages: int = 256, max_requests: int = 8, max_seq_len: Optional[int] = None, model=None,
                 use_graphs: bool = True, release_window_pages: bool = True,
                 max_step_tokens: Optional[int] = None):
        self.config = config
        self.rt = rt
        self.spec = config.model_spec()
        self.model = model if model is not None else build_model(self.spec)
        self.model.bind(weights, rt)
        self.page_size = int(page_size)
        if max_seq_len is None:
            max_seq_len = self.spec.max_positions if self.spec.max_positions > 0 else num_pages * page_size
        self.max_seq_len = int(max_seq_len)
        self.max_requests = int(max_requests)
        self.use_graphs = bool(use_graphs) and self.model.graph_safe()
        # False: windowed groups keep every page until the request ends (for differential tests of the release)
        self.release_window_pages = bool(release_window_pages)
        # the most tokens of one request that a step will bring, if the caller promises one (the scheduler's budget):
        # windowed groups then get pools sized by window + step instead of by context
        self.max_step_tokens = max_step_tokens
        self._lay_out_cache(int(num_pages))

    @classmethod
    def from_directory(cls, model_dir: str, dtype="bfloat16", device: str = "cuda:0", **kw) -> "ModelRunner":
        config = config_from_directory(model_dir)
        rt = Runtime(dtype, device)
        model = build_model(config.model_spec())
        weights = load_weights(model, model_dir, rt)
        return cls(config, weights, rt, model=model, **kw)

    # ---- cache memory ------------------------------------------------------
    def _lay_out_cache(self, num_pages: int) -> None:
        """Memory for what the parts keep between steps, from their own descriptions: per page group (the owners
        of equal `CacheNeed`s) and array one tensor [owners, pages, heads, page_size, width] (the last two swapped
        for a transposed array), per state one tensor [requests, *shape]."""
        plan = self.model.cache_plan()
        rt = self.rt
        needs: List = []                        # distinct CacheNeed, one page group each
        owners: List[List[Tuple[int, str]]] = []  # per group the (schedule entry, part name) that own pages in it
        for i, (keeps, cache_from) in enumerate(plan):
            if cache_from is not None:
                continue
            for name, (need, _state) in keeps.items():
                if need is None:
                    continue
                if need not in needs:
                    needs.append(need)
                    owners.append([])
                owners[needs.index(need)].append((i, name))
        self.group_needs, self.group_owners = needs, owners
        self.group_pages = [self.pages_of_group(n, num_pages) for n in needs]
        dtype_of = lambda name: rt.dtype if name is None else {"float32": torch.float32, "bfloat16": torch.bfloat16}[name]
        self.pages: List[Dict[str, torch.Tensor]] = []
        for g, need in enumerate(needs):
            arrays = {}
            for a in need.arrays:
                shape = (a.heads, a.width, self.page_size) if a.transposed else (a.heads, self.page_size, a.width)
                arrays[a.name] = torch.zeros((len(owners[g]), self.group_pages[g]) + shape, dtype=dtype_of(a.dtype),
                                             device=rt.device)
            self.pages.append(arrays)
        self.bindings: List[Dict[str, CacheBinding]] = []
        for i, (keeps, cache_from) in enumerate(plan):
            bound: Dict[str, CacheBinding] = {}
            for name, (need, state) in keeps.items():
                b = CacheBinding()
                if need is not None:
                    src = i if cache_from is None else cache_from
                    src_need = plan[src][0].get(name, (None, None))[0]
                    if src_need != need:
                        raise ValueError(f"schedule entry {i} reads the cache that entry {src} keeps for its part "
                                         f"{name!r}, whose layout differs")
                    g = needs.index(need)
                    j = owners[g].index((src, name))
                    b.group, b.writes = g, cache_from is None
                    b.arrays = {a.name: self.pages[g][a.name][j] for a in need.arrays}
                if state is not None:
                    b.state = torch.zeros((self.max_requests,) + tuple(state.shape), device=rt.device,
                                          dtype=STATE_TYPES[state.dtype])
                bound[name] = b
            self.bindings.append(bound)
        self._states = [b.state for bound in self.bindings for b in bound.values() if b.state is not None]
        self.cache = CacheManager([GroupLayout(n.window, self.release_window_pages) for n in needs],
                                  self.group_pages, self.page_size, self.max_requests, self.max_seq_len,
                                  self.max_step_tokens)
        self._graphs: Dict[Tuple[int, int], "_DecodeGraph"] = {}
        self._graph_uses: Dict[Tuple[int, int], int] = {}
        self._graph_logits: Optional[torch.Tensor] = None
        self.max_graphs = 128   # the least recently replayed shape goes when there are more
        self.capture_after = 3  # (1: every shape is captured at its first step; see _graph_step)
        self._graph_pool = None
        self._capture_stream = None

    def pages_of_group(self, need, num_pages: int) -> int:
        """A group that keeps every token gets `num_pages`; a windowed one that gives passed pages back, when the
        largest step is known, no more than it can ever hold."""
        if need.window > 0 and self.release_window_pages and self.max_step_tokens:
            return min(num_pages, pages_for_window(need.window, self.page_size, self.max_requests, self.max_step_tokens))
        return num_pages

    def kv_bytes_per_token(self) -> int:
        """Bytes that one token takes in the pages of all groups."""
        return sum(t.shape[0] * t.shape[2] * t.shape[3] * t.shape[4] // self.page_size * t.element_size()
                   for arrays in self.pages for t in arrays.values())

    def page_bytes(self, group: int) -> int:
        """Bytes of one page of a group, all its owners' arrays together."""
        return sum(t.shape[0] * t.shape[2] * t.shape[3] * t.shape[4] * t.element_size()
                   for t in self.pages[group].values())

    def cache_bytes(self, num_pages: int) -> int:
        """Bytes of all pools if the groups that keep every token get `num_pages` pages."""
        return sum(self.pages_of_group(n, num_pages) * self.page_bytes(g) for g, n in enumerate(self.group_needs))

    @property
    def keeps_state(self) -> bool:
        """Whether some part keeps a block of state per request (which a step advances, so that a step cannot simply
        be run again)."""
        return bool(self._states)

    # ---- the step ------------------------------------------------------------
    def step(self, batch: StepBatch) -> torch.Tensor:
        """Run the batch; float32 logits [len(batch.logits_rows), vocab] on the device."""
        batch.validate(self.spec.vocab_size, [p.num_pages for p in self.cache.pools], self.page_size)
        if batch.num_tokens == 0:
            return self.rt.empty((0, self.spec.vocab_size), torch.float32)
        self._zero_fresh_state(batch)
        if self.use_graphs and batch.one_token_each:
            return self._graph_step(batch)
        return self.model.forward(self._upload(batch), self.bindings)

    def _zero_fresh_state(self, batch: StepBatch) -> None:
        """State slots of requests that start at position 0 in this step are cleared (before the step is
        launched, so also before a captured step is replayed)."""
        if not self._states:
            return
        first = batch.q_start[:-1]
        brings = batch.q_start[1:] > first
        starts = np.zeros(batch.num_requests, dtype=bool)
        starts[brings] = batch.positions[first[brings]] == 0
        if starts.any():
            slots = torch.from_numpy(batch.state_slots[starts].astype(np.int64)).to(self.rt.device)
            for state in self._states:
                state.index_fill_(0, slots, 0)

    def _context(self, dev: torch.Tensor, sizes: List[int], batch: StepBatch) -> StepContext:
        views, at = [], 0
        for n in sizes:
            views.append(dev[at:at + n])
            at += n
        T, S = batch.num_tokens, batch.num_requests
        G = len(batch.slots)
        tables = [views[N_FIXED + G + g].view(S, -1) for g in range(G)]
        return StepContext(rt=self.rt, num_tokens=T, num_requests=S, token_ids=views[0], positions=views[1],
                           seq_of_token=views[2], q_start=views[3], seq_lens=views[4], state_slots=views[5],
                           logits_rows=views[6], slots=views[N_FIXED:N_FIXED + G], block_tables=tables, host=batch,
                           one_token_each=batch.one_token_each)

    def _upload(self, batch: StepBatch) -> StepContext:
        sizes, flat = _pack(batch)
        return self._context(torch.from_numpy(flat).to(self.rt.device), sizes, batch)

    # ---- graphs for one-token-per-request steps ---------------------------------
    def _shared_logits(self, rows: int) -> torch.Tensor:
        """The first `rows` rows of the buffer that captured steps leave their logits in."""
        if self._graph_logits is None:
            self._graph_logits = torch.empty((self.max_requests, self.spec.vocab_size), dtype=torch.float32,
                                             device=self.rt.device)
        return self._graph_logits[:rows]

    def _graph_step(self, batch: StepBatch) -> torch.Tensor:
        S = batch.num_requests
        longest = int(batch.seq_lens.max())
        bucket = 1 << max(longest - 1, 0).bit_length()  # context rounded up to a power of two
        key = (S, bucket)
        graph = self._graphs.get(key)
        if graph is None:
            # A shape is captured when it comes for the `capture_after`-th time: a capture costs as much as three
            # steps (a warm-up run, the recording, the instantiation: 13 ms at 24 layers), and a batch that drains
            # passes through many shapes once or twice (96 requests of mixed lengths, 64 at a time: 48 shapes in
            # 150 steps, 12 of them seen three times).
            uses = self._graph_uses[key] = self._graph_uses.get(key, 0) + 1
            if uses < self.capture_after:
                # kernel by kernel, with the plans that the recorded step of this shape will have: a request's
                # results then do not depend on how often the shape has come before
                ctx = self._upload(batch)
                self.plan_one_token_step(ctx, S, bucket)
                return self.model.forward(ctx, self.bindings)
            if len(self._graphs) >= self.max_graphs:
                del self._graphs[next(iter(self._graphs))]
            graph = _DecodeGraph(self, batch, bucket)
        self._graphs.pop(key, None)
        self._graphs[key] = graph  # (the dict keeps the order of use: the first key is the least recently used)
        return graph.run(batch)

    def plan_one_token_step(self, ctx: StepContext, requests: int, longest: int) -> None:
        """Every part leaves in `ctx.memo` what it plans on the host for a step of one token per request
        (`Part.capture_plan`); the runner itself knows none of these plans."""
        for part in self.model.all_parts():
            plan = getattr(part, "capture_plan", None)
            if plan is not None:
                plan(ctx, requests, longest)

    # ---- convenience over the cache manager -----------------------------------
    def add_request(self, rid: Hashable) -> None:
        self.cache.add(rid)

    def end_request(self, rid: Hashable) -> None:
        self.cache.free(rid)

    def run_entries(self, entries: Sequence[Entry]) -> torch.Tensor:
        """Reserve pages, run one step, commit.  Raises `OutOfPages` before anything ran."""
        batch = build_step_batch(self.cache, entries)
        logits = self.step(batch)
        for rid, tokens, _ in entries:
            self.cache.commit(rid, len(tokens))
        return logits


class _DecodeGraph:
    """One captured step for `S` requests of one token each, contexts up to `bucket`."""

    def __init__(self, runner: ModelRunner, batch: StepBatch, bucket: int):
        rt = runner.rt
        S = batch.num_requests
        all_rows = self._with_all_rows(batch)
        sizes, flat = _pack(all_rows)
        self.sizes = sizes
        self.host = torch.empty(flat.size, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.empty(flat.size, dtype=torch.int32, device=rt.device)
        self.copied = torch.cuda.Event()
        self._fill(flat)
        ctx = runner._context(self.dev, sizes, all_rows)
        ctx.host = None  # nothing may plan from host data inside the capture:
        runner.plan_one_token_step(ctx, S, bucket)  # what the parts plan on the host, they plan here, once
        plans = dict(ctx.memo)
        self.ctx = ctx
        # The warm-up run really executes the step.  What it appends to the pages the replay writes again, the same
        # values to the same places; per-request state, though, would be advanced twice, so it is put back.
        kept = [state.clone() for state in runner._states]
        self.logits = runner._shared_logits(S)  # (allocated before the capture, outside the graphs' pool)
        # Warm-up and capture run on one stream that all of the runner's graphs share: what a library keeps per
        # stream (the dense products' workspace) is there before the capture, and once for all graphs.
        if runner._capture_stream is None:
            runner._capture_stream = torch.cuda.Stream()
        side = runner._capture_stream
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            runner.model.forward(ctx, runner.bindings)  # warm-up: library plans, allocator
            ctx.memo = dict(plans)  # (what the warm-up run memoised was made outside the recording)
            for state, before in zip(runner._states, kept):
                state.copy_(before)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        # (capture_begin / capture_end themselves: the context manager that wraps them also collects Python's garbage
        # and gives the allocator's cached blocks back first, tens of milliseconds per capture in a running engine)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            if runner._graph_pool is None:
                self.graph.capture_begin()
            else:
                self.graph.capture_begin(pool=runner._graph_pool)
            try:
                # The step's logits end in a buffer that all of the runner's graphs share, as the last node of the
                # graph: what the capture allocated is then free for the next capture (the graphs share a memory
                # pool), and a graph holds nothing of the size of requests x vocabulary for itself.
                logits = runner.model.forward(ctx, runner.bindings)
                self.logits.copy_(logits)
                del logits
            finally:
                self.graph.capture_end()
        torch.cuda.current_stream().wait_stream(side)
        if runner._graph_pool is None:
            runner._graph_pool = self.graph.pool()

    @staticmethod
    def _with_all_rows(batch: StepBatch) -> StepBatch:
        return StepBatch(batch.token_ids, batch.positions, batch.seq_of_token, batch.q_start, batch.seq_lens,
                         batch.state_slots, np.arange(batch.num_tokens, dtype=np.int32), batch.slots,
                         batch.block_tables, batch.request_ids)

    def _fill(self, flat: np.ndarray) -> None:
        self.copied.synchronize()  # the pinned buffer is free again
        self.host_np[:] = flat
        self._send()

    def _send(self) -> None:
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def run(self, batch: StepBatch) -> torch.Tensor:
        T = batch.num_tokens
        self.copied.synchronize()  # the pinned buffer is free again
        sizes, _ = _pack(self._with_all_rows(batch), out=self.host_np)
        if sizes != self.sizes:
            raise RuntimeError("a captured step was given a batch of another shape")
        self._send()
        self.graph.replay()
        rows = batch.logits_rows
        if len(rows) == T and (T == 0 or (rows[0] == 0 and rows[-1] == T - 1 and np.all(rows[1:] > rows[:-1]))):
            return self.logits.clone()
        return self.logits[torch.from_numpy(rows.astype(np.int64)).to(self.logits.device)]
