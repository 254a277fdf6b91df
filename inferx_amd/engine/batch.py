"""The flat description of one step: the only thing that crosses from the
scheduling side (scheduler, trace replay) to the model.

Plain int32 arrays, as in the reference's `ForwardBatch`
(`include/inferx/model/forward_batch.h:20-124`; checks `forward_batch.cc:5-93`).
Rows are grouped by request in the order of `entries`, positions ascend within
a request.  Each page group has its own `slots` and `block_table`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Hashable, List, Sequence, Tuple

import numpy as np

from ..cache.manager import CacheManager, RESERVE_OK


class BatchError(ValueError):
    pass


class OutOfPages(RuntimeError):
    """Pages (or context) ran out while a step's batch was being put together."""

    def __init__(self, rid, reason: str):
        super().__init__(f"request {rid!r}: {reason}")
        self.rid, self.reason = rid, reason


@dataclass
class StepBatch:
    token_ids: np.ndarray      # [T]
    positions: np.ndarray      # [T]
    seq_of_token: np.ndarray   # [T]
    q_start: np.ndarray        # [S + 1] first row of each request, then T
    seq_lens: np.ndarray       # [S] tokens in the cache once this step has run
    state_slots: np.ndarray    # [S]
    logits_rows: np.ndarray    # [R] rows whose logits are wanted
    slots: List[np.ndarray]          # per group [T]
    block_tables: List[np.ndarray]   # per group [S, max_blocks], -1 where no page is held
    request_ids: List[Hashable]

    @property
    def num_tokens(self) -> int:
        return int(self.token_ids.shape[0])

    @property
    def num_requests(self) -> int:
        return int(self.seq_lens.shape[0])

    def validate(self, vocab_size: int, pages_per_group: Sequence[int], page_size: int) -> None:
        T, S = self.num_tokens, self.num_requests
        for name in ("positions", "seq_of_token"):
            if getattr(self, name).shape != (T,):
                raise BatchError(f"{name} must hold one entry per token")
        if self.q_start.shape != (S + 1,) or self.q_start[0] != 0 or self.q_start[-1] != T:
            raise BatchError("q_start must run from 0 to the number of tokens")
        if T and (self.token_ids.min() < 0 or self.token_ids.max() >= vocab_size):
            bad = self.token_ids[(self.token_ids < 0) | (self.token_ids >= vocab_size)][0]
            raise BatchError(f"token id {int(bad)} is outside the vocabulary of {vocab_size}")
        n = self.q_start[1:].astype(np.int64) - self.q_start[:-1]
        if S and n.min() < 0:
            raise BatchError("q_start must not descend")
        first = self.seq_lens.astype(np.int64) - n
        if S and first.min() < 0:
            s = int(np.argmax(first < 0))
            raise BatchError(f"request {s}: more tokens in the step than in the sequence")
        if T:
            want_seq = np.repeat(np.arange(S, dtype=np.int64), n)
            want_pos = np.arange(T, dtype=np.int64) - np.repeat(self.q_start[:-1].astype(np.int64), n) + np.repeat(first, n)
            bad = (self.seq_of_token != want_seq) | (self.positions != want_pos)
            if bad.any():
                s = int(want_seq[int(np.argmax(bad))])
                raise BatchError(f"request {s}: rows must be grouped, positions contiguous and ending at seq_len - 1")
        if len(self.logits_rows) and (self.logits_rows.min() < 0 or self.logits_rows.max() >= T):
            raise BatchError("logits_rows points outside the step's tokens")
        if len(self.slots) != len(pages_per_group) or len(self.block_tables) != len(pages_per_group):
            raise BatchError("one slots array and one block table per page group are needed")
        for g, pages in enumerate(pages_per_group):
            sl, bt = self.slots[g], self.block_tables[g]
            if sl.shape != (T,) or bt.ndim != 2 or bt.shape[0] != S:
                raise BatchError(f"group {g}: slots or block table have the wrong shape")
            if T and (sl.min() < 0 or sl.max() >= pages * page_size):
                raise BatchError(f"group {g}: a slot lies outside the pool")
            if bt.size and bt.max() >= pages:
                raise BatchError(f"group {g}: the block table names a page outside the pool")
            # every slot written this step is reachable through this step's table
            if T:
                page_of = bt[self.seq_of_token, self.positions // page_size]
                if np.any(page_of * page_size + self.positions % page_size != sl):
                    raise BatchError(f"group {g}: a slot is not covered by the block table")


Entry = Tuple[Hashable, Sequence[int], Sequence[int]]  # request id, its next tokens, wanted places among them


def build_step_batch(cache: CacheManager, entries: Sequence[Entry]) -> StepBatch:
    """Reserve pages for every entry and lay the step out flat.  On a shortage
    nothing of this step stays reserved beyond what earlier steps held... the
    caller decides what to do (`OutOfPages`); commit happens after the step ran."""
    seen = set()
    for rid, tokens, want in entries:
        if rid in seen:
            raise BatchError(f"request {rid!r} appears twice in one step")
        seen.add(rid)
        if rid not in cache:
            raise BatchError(f"request {rid!r} is not live")
        for w in want:
            if not 0 <= w < len(tokens):
                raise BatchError(f"request {rid!r}: wanted place {w} is outside its {len(tokens)} tokens")
    for rid, tokens, _ in entries:
        status = cache.reserve(rid, cache.cached(rid) + len(tokens))
        if status != RESERVE_OK:
            raise OutOfPages(rid, status)

    G = len(cache.groups)
    P = cache.page_size
    S = len(entries)
    T = sum(len(tokens) for _, tokens, _ in entries)
    token_ids = np.zeros(T, np.int32)
    positions = np.zeros(T, np.int32)
    seq_of_token = np.zeros(T, np.int32)
    q_start = np.zeros(S + 1, np.int32)
    seq_lens = np.zeros(S, np.int32)
    state_slots = np.zeros(S, np.int32)
    slots = [np.zeros(T, np.int32) for _ in range(G)]
    tables = [np.full((S, cache.max_blocks), -1, np.int32) for _ in range(G)]
    logits_rows: List[int] = []
    row = 0
    for s, (rid, tokens, want) in enumerate(entries):
        n = len(tokens)
        first = cache.cached(rid)
        q_start[s] = row
        seq_lens[s] = first + n
        state_slots[s] = cache.slot_of(rid)
        token_ids[row:row + n] = np.asarray(tokens, dtype=np.int64)
        pos = np.arange(first, first + n, dtype=np.int32)
        positions[row:row + n] = pos
        seq_of_token[row:row + n] = s
        for g in range(G):
            blocks = np.asarray(cache.block_row(rid, g), dtype=np.int32)
            tables[g][s, :len(blocks)] = blocks
            if n:
                slots[g][row:row + n] = blocks[pos // P] * P + pos % P
        logits_rows.extend(row + w for w in want)
        row += n
    q_start[S] = row
    return StepBatch(token_ids, positions, seq_of_token, q_start, seq_lens, state_slots,
                     np.asarray(logits_rows, dtype=np.int32), slots, tables, [e[0] for e in entries])
