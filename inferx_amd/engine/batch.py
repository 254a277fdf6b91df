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

import ctypes

from ..cache.manager import RESERVE_CONTEXT_FULL, RESERVE_POOL_EMPTY, CacheManager


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
    laid_out_by_manager: bool = False  # True: the host library built it, so only the token ids are unchecked

    @property
    def num_tokens(self) -> int:
        return int(self.token_ids.shape[0])

    @property
    def num_requests(self) -> int:
        return int(self.seq_lens.shape[0])

    @property
    def one_token_each(self) -> bool:
        """Every request of the step brings exactly one token (a request may also bring none, so equal counts of
        tokens and requests do not say so)."""
        return self.num_tokens == self.num_requests and bool(np.all(self.q_start[1:] - self.q_start[:-1] == 1))

    def validate(self, vocab_size: int, pages_per_group: Sequence[int], page_size: int) -> None:
        T, S = self.num_tokens, self.num_requests
        if T and (self.token_ids.min() < 0 or self.token_ids.max() >= vocab_size):
            bad = self.token_ids[(self.token_ids < 0) | (self.token_ids >= vocab_size)][0]
            raise BatchError(f"token id {int(bad)} is outside the vocabulary of {vocab_size}")
        if self.laid_out_by_manager:
            return
        for name in ("positions", "seq_of_token"):
            if getattr(self, name).shape != (T,):
                raise BatchError(f"{name} must hold one entry per token")
        if self.q_start.shape != (S + 1,) or self.q_start[0] != 0 or self.q_start[-1] != T:
            raise BatchError("q_start must run from 0 to the number of tokens")
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
    """Reserve pages for every entry and lay the step out flat (done by the host library in one call).  On a
    shortage `OutOfPages` is raised: entries before the failing one keep what they reserved, nothing was run,
    and the caller decides what to do.  Commit happens after the step ran."""
    S = len(entries)
    G = len(cache.groups)
    for rid, _, _ in entries:
        if rid not in cache:
            raise BatchError(f"request {rid!r} is not live")
    rids = np.fromiter((cache._ids[e[0]] for e in entries), dtype=np.int64, count=S)
    n_tokens = np.fromiter((len(e[1]) for e in entries), dtype=np.int32, count=S)
    n_want = np.fromiter((len(e[2]) for e in entries), dtype=np.int32, count=S)
    T, R = int(n_tokens.sum()), int(n_want.sum())
    tokens_flat = np.fromiter((t for e in entries for t in e[1]), dtype=np.int64, count=T)
    if T and (tokens_flat.min() < -(1 << 31) or tokens_flat.max() >= (1 << 31)):
        raise BatchError("a token id does not fit 32 bits")
    tokens_flat = tokens_flat.astype(np.int32)
    want_flat = np.fromiter((w for e in entries for w in e[2]), dtype=np.int32, count=R)
    token_ids, positions, seq_of_token = (np.empty(T, np.int32) for _ in range(3))
    q_start, seq_lens, state_slots = np.empty(S + 1, np.int32), np.empty(S, np.int32), np.empty(S, np.int32)
    logits_rows = np.empty(R, np.int32)
    slots = np.empty((G, T), np.int32)
    tables = np.empty((G, S, cache.max_blocks), np.int32)
    failed = ctypes.c_int(0)
    p32 = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    rc = cache._lib.ixh_build_batch(
        cache._h, S, rids.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), p32(n_tokens), p32(tokens_flat),
        p32(n_want), p32(want_flat), p32(token_ids), p32(positions), p32(seq_of_token), p32(q_start), p32(seq_lens),
        p32(state_slots), p32(logits_rows), p32(slots), p32(tables), ctypes.byref(failed))
    if rc != 0:
        rid = entries[failed.value][0] if 0 <= failed.value < S else None
        if rc in (1, 2):
            raise OutOfPages(rid, RESERVE_POOL_EMPTY if rc == 1 else RESERVE_CONTEXT_FULL)
        raise BatchError(f"request {rid!r} " + cache._lib.ixh_cache_error(cache._h).decode("utf-8", "replace"))
    return StepBatch(token_ids, positions, seq_of_token, q_start, seq_lens, state_slots, logits_rows,
                     [slots[g] for g in range(G)], [tables[g] for g in range(G)], [e[0] for e in entries],
                     laid_out_by_manager=True)
