"""The step function and the memory it runs on.

`ModelRunner` owns the model (parts with their weights bound), the cache
memory (pages of keys and values per group, state slots) and the host-side
`CacheManager`.  `step(batch)` runs exactly the tokens the batch brings, as one
batch, against the cache that earlier steps left, and returns float32 logits
at the wanted rows (reference: Qwen2Model::Step, src/model/qwen2.cc:2246-2277;
PrepareBatchInputs :564-817).  It holds no policy: who runs, in which portions,
and what happens when pages run out is decided above it (scheduler, replay).
"""
from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, GroupLayout
from ..config import config_from_directory
from ..parts import build_model
from ..weights import load_weights
from .batch import Entry, StepBatch, build_step_batch
from .runtime import CacheBinding, Runtime, StepContext


class ModelRunner:
    def __init__(self, config, weights: Dict[str, torch.Tensor], rt: Runtime, *, page_size: int = 16,
                 num_pages: int = 256, max_requests: int = 8, max_seq_len: Optional[int] = None, model=None):
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
        plan = self.model.cache_plan()
        needs: List = []           # distinct CacheNeed, one page group each
        owners: List[List[int]] = []
        for i, (need, _state, cache_from) in enumerate(plan):
            if need is None or cache_from is not None:
                continue
            if need not in needs:
                needs.append(need)
                owners.append([])
            owners[needs.index(need)].append(i)
        self.group_needs = needs
        rt = self.rt
        self.kv: List[torch.Tensor] = [
            torch.zeros((len(owners[g]), 2, num_pages, n.kv_heads, self.page_size, n.head_dim), dtype=rt.dtype,
                        device=rt.device) for g, n in enumerate(needs)]
        self.bindings: List[CacheBinding] = []
        for i, (need, state, cache_from) in enumerate(plan):
            b = CacheBinding()
            if need is not None:
                src = i if cache_from is None else cache_from
                src_need = plan[src][0]
                if src_need != need:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {src}, whose layout differs")
                g = needs.index(need)
                j = owners[g].index(src)
                n_ = needs[g]
                b.group, b.k, b.writes = g, self.kv[g][j, 0], cache_from is None
                # values are kept transposed within a page: [pages, kv_heads, head_dim, page_size]
                b.v = self.kv[g][j, 1].view(-1, n_.kv_heads, n_.head_dim, self.page_size)
            if state is not None:
                b.state = torch.zeros((self.max_requests,) + tuple(state.shape), dtype=torch.float32,
                                      device=rt.device)
            self.bindings.append(b)
        self.cache = CacheManager([GroupLayout(n.window) for n in needs], [num_pages] * len(needs), self.page_size,
                                  self.max_requests, self.max_seq_len)

    def kv_bytes_per_token(self) -> int:
        size = torch.empty((), dtype=self.rt.dtype).element_size()
        return sum(t.shape[0] * 2 * n.kv_heads * n.head_dim * size for t, n in zip(self.kv, self.group_needs))

    # ---- the step ------------------------------------------------------------
    def step(self, batch: StepBatch) -> torch.Tensor:
        """Run the batch; float32 logits [len(batch.logits_rows), vocab] on the device."""
        batch.validate(self.spec.vocab_size, [p.num_pages for p in self.cache.pools], self.page_size)
        ctx = self._upload(batch)
        for b in self.bindings:
            if b.state is not None:
                fresh = [int(batch.state_slots[s]) for s in range(batch.num_requests)
                         if batch.q_start[s + 1] > batch.q_start[s] and batch.positions[batch.q_start[s]] == 0]
                if fresh:
                    b.state[fresh] = 0
        return self.model.forward(ctx, self.bindings)

    def _upload(self, batch: StepBatch) -> StepContext:
        T, S = batch.num_tokens, batch.num_requests
        parts = [batch.token_ids, batch.positions, batch.seq_of_token, batch.q_start, batch.seq_lens,
                 batch.state_slots, batch.logits_rows] + list(batch.slots) + [t.reshape(-1) for t in batch.block_tables]
        sizes = [p.size for p in parts]
        flat = np.concatenate([np.ascontiguousarray(p, dtype=np.int32).reshape(-1) for p in parts]) \
            if sum(sizes) else np.zeros(0, np.int32)
        dev = torch.from_numpy(flat).to(self.rt.device)
        views, at = [], 0
        for n in sizes:
            views.append(dev[at:at + n])
            at += n
        G = len(batch.slots)
        tables = [views[7 + G + g].view(S, -1) for g in range(G)]
        return StepContext(rt=self.rt, num_tokens=T, num_requests=S, token_ids=views[0], positions=views[1],
                           seq_of_token=views[2], q_start=views[3], seq_lens=views[4], state_slots=views[5],
                           logits_rows=views[6], slots=views[7:7 + G], block_tables=tables, host=batch)

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
