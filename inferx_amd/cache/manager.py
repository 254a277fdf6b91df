"""Host-side bookkeeping of what requests keep between steps.  Touches no GPU.

  PagePool      fixed number of pages, LIFO free list, double-free check
                (reference: KvBlockPool, src/core/kv_cache.cc:58-104)
  CacheManager  per request: tokens cached so far, one block list per page
                group, one state slot
                (reference: BlockTable, include/inferx/core/kv_cache.h:158-186;
                Reserve / ReleaseBlocks, src/scheduler/scheduler.cc:99-111, 170-190)

A page group is a set of cache-owning layer executions with the same need (kv
heads, head size, window).  Every group has pages of its own: its own pool, its
own block list per request.  A group with window W gives a page back as soon as
no query at or after the request's next position can read it: page j (tokens
[j*P, (j+1)*P)) is dead once (j+1)*P <= cached + 1 - W.  The reference keeps
every token of its windowed layers (src/model/gpt_oss.cc:259-262); releasing
is this engine's own rule.

State slots are fixed-size blocks per request for mixers that carry state of
their own; the manager hands out slot numbers, the runner owns the memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence


class CacheError(RuntimeError):
    """Misuse of the cache manager (unknown request, double free, ...)."""


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))  # page 0 is handed out first
        self._is_free = [True] * num_pages

    @property
    def free_pages(self) -> int:
        return len(self._free)

    @property
    def used_pages(self) -> int:
        return self.num_pages - len(self._free)

    def allocate(self) -> Optional[int]:
        if not self._free:
            return None
        page = self._free.pop()
        self._is_free[page] = False
        return page

    def release(self, page: int) -> None:
        if not 0 <= page < self.num_pages:
            raise CacheError(f"page {page} is outside the pool of {self.num_pages}")
        if self._is_free[page]:
            raise CacheError(f"page {page} freed twice")
        self._is_free[page] = True
        self._free.append(page)


@dataclass(frozen=True)
class GroupLayout:
    """One page group: `window` 0 keeps every token, W > 0 only the last W."""

    window: int = 0


@dataclass
class _Request:
    cached: int = 0
    reserved: int = 0  # tokens that pages have been reserved for (>= cached)
    slot: int = -1
    blocks: List[List[int]] = field(default_factory=list)  # per group, by logical page; -1 = given back


RESERVE_OK, RESERVE_POOL_EMPTY, RESERVE_CONTEXT_FULL = "ok", "pool_empty", "context_full"


class CacheManager:
    def __init__(self, groups: Sequence[GroupLayout], pages_per_group: Sequence[int], page_size: int,
                 max_requests: int, max_seq_len: int):
        if page_size <= 0 or max_requests <= 0 or max_seq_len <= 0:
            raise CacheError("page_size, max_requests and max_seq_len must be positive")
        if len(groups) != len(pages_per_group):
            raise CacheError("one page count per group is needed")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_seq_len = max_seq_len
        self.max_blocks = -(-max_seq_len // page_size)
        self.pools = [PagePool(n) for n in pages_per_group]
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[Hashable, _Request] = {}

    # ---- requests -------------------------------------------------------
    def __contains__(self, rid) -> bool:
        return rid in self._requests

    def live_requests(self):
        return list(self._requests)

    def _get(self, rid) -> _Request:
        try:
            return self._requests[rid]
        except KeyError:
            raise CacheError(f"unknown request {rid!r}") from None

    def can_add(self) -> bool:
        return bool(self._free_slots)

    def add(self, rid) -> int:
        """Start a request: takes a state slot, no pages yet.  Returns the slot."""
        if rid in self._requests:
            raise CacheError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise CacheError(f"all {self.max_requests} request slots are taken")
        slot = self._free_slots.pop()
        self._requests[rid] = _Request(slot=slot, blocks=[[] for _ in self.groups])
        return slot

    def free(self, rid) -> None:
        """End a request: every page and the state slot go back."""
        req = self._get(rid)
        self._drop_pages(req)
        self._free_slots.append(req.slot)
        del self._requests[rid]

    def reset(self, rid) -> None:
        """Preemption by recomputation: pages go back, the request starts over at
        position 0 and keeps its slot (reference: Preempt, scheduler.cc:206-229)."""
        req = self._get(rid)
        self._drop_pages(req)
        req.cached = req.reserved = 0

    def _drop_pages(self, req: _Request) -> None:
        for g, blocks in enumerate(req.blocks):
            for page in blocks:
                if page >= 0:
                    self.pools[g].release(page)
            blocks.clear()

    # ---- pages ----------------------------------------------------------
    def cached(self, rid) -> int:
        return self._get(rid).cached

    def slot_of(self, rid) -> int:
        return self._get(rid).slot

    def _first_live_page(self, group: int, cached: int) -> int:
        w = self.groups[group].window
        if w <= 0:
            return 0
        return max(0, cached + 1 - w) // self.page_size

    def _release_passed(self, req: _Request) -> None:
        for g, blocks in enumerate(req.blocks):
            first = min(self._first_live_page(g, req.cached), len(blocks))
            for j in range(first):
                if blocks[j] >= 0:
                    self.pools[g].release(blocks[j])
                    blocks[j] = -1

    def pages_short(self, rid, new_len: int) -> List[int]:
        """Per group, how many pages a growth to `new_len` tokens would need beyond what is free."""
        req = self._get(rid)
        short = []
        for g, blocks in enumerate(req.blocks):
            need = max(0, -(-new_len // self.page_size) - len(blocks))
            # pages of this request that the window has passed come back first
            first = min(self._first_live_page(g, req.cached), len(blocks))
            coming = sum(1 for j in range(first) if blocks[j] >= 0)
            short.append(max(0, need - self.pools[g].free_pages - coming))
        return short

    def reserve(self, rid, new_len: int) -> str:
        """Make sure pages exist for tokens [0, new_len) (as far as each group's
        window still needs them).  All groups or nothing."""
        req = self._get(rid)
        if new_len > self.max_seq_len:
            return RESERVE_CONTEXT_FULL
        if new_len <= req.reserved:
            return RESERVE_OK
        self._release_passed(req)
        want_pages = -(-new_len // self.page_size)
        needs = [max(0, want_pages - len(b)) for b in req.blocks]
        if any(n > self.pools[g].free_pages for g, n in enumerate(needs)):
            return RESERVE_POOL_EMPTY
        for g, n in enumerate(needs):
            for _ in range(n):
                req.blocks[g].append(self.pools[g].allocate())
        req.reserved = new_len
        return RESERVE_OK

    def commit(self, rid, tokens: int) -> None:
        """`tokens` more tokens are now in the cache."""
        req = self._get(rid)
        if tokens < 0 or req.cached + tokens > req.reserved:
            raise CacheError(f"request {rid!r}: commit of {tokens} tokens beyond the {req.reserved} reserved")
        req.cached += tokens
        self._release_passed(req)

    def block_row(self, rid, group: int) -> List[int]:
        """The request's pages in this group by logical page number, -1 where none is held."""
        return self._get(rid).blocks[group]

    def slot_index(self, rid, group: int, position: int) -> int:
        """Flat index page * page_size + offset of the token at `position`."""
        blocks = self._get(rid).blocks[group]
        j = position // self.page_size
        if j >= len(blocks) or blocks[j] < 0:
            raise CacheError(f"request {rid!r}: no page holds position {position} in group {group}")
        return blocks[j] * self.page_size + position % self.page_size

    # ---- invariants (used by tests and by debug runs) ---------------------
    def check(self) -> None:
        """Every page is free or held exactly once; every slot likewise."""
        for g, pool in enumerate(self.pools):
            held = [p for r in self._requests.values() for p in r.blocks[g] if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError(f"group {g}: a page is held twice")
            if any(pool._is_free[p] for p in held):
                raise CacheError(f"group {g}: a held page is on the free list")
            if len(held) + pool.free_pages != pool.num_pages:
                raise CacheError(f"group {g}: {pool.num_pages - len(held) - pool.free_pages} pages lost")
            if len(set(pool._free)) != len(pool._free):
                raise CacheError(f"group {g}: a page is on the free list twice")
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots + self._free_slots)) != self.max_requests or len(slots) + len(self._free_slots) != self.max_requests:
            raise CacheError("a state slot is lost or held twice")
