"""Host-side bookkeeping of what requests keep between steps.  Touches no GPU.

  PagePool      fixed number of pages, LIFO free list, double-free check
                (reference: KvBlockPool, src/core/kv_cache.cc:58-104)
  CacheManager  per request: tokens cached so far, one block list per page
                group, one state slot
                (reference: BlockTable, include/inferx/core/kv_cache.h:158-186;
                Reserve / ReleaseBlocks, src/scheduler/scheduler.cc:99-111, 170-190)

The bookkeeping itself is C++ (`inferx_amd/csrc/host/cache.cc`, built into
libinferx_host.so with the host compiler); these classes are its Python face.

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

import ctypes
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence

from ..csrc import build as _build


class CacheError(RuntimeError):
    """Misuse of the cache manager (unknown request, double free, ...)."""


_configured = False


def host_lib():
    """libinferx_host.so with its argument types declared."""
    global _configured
    lib = _build.load_host()
    if not _configured:
        i32p, i64p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64)
        vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        sig = {
            "ixh_cache_create": (vp, [ci, i32p, i32p, ci, ci, i64, i64]),
            "ixh_cache_destroy": (None, [vp]),
            "ixh_cache_error": (ctypes.c_char_p, [vp]),
            "ixh_cache_max_blocks": (ci, [vp]),
            "ixh_cache_add": (ci, [vp, i64]),
            "ixh_cache_free": (ci, [vp, i64]),
            "ixh_cache_reset": (ci, [vp, i64]),
            "ixh_cache_reserve": (ci, [vp, i64, i64]),
            "ixh_cache_commit": (ci, [vp, i64, i64]),
            "ixh_cache_cached": (i64, [vp, i64]),
            "ixh_cache_slot": (ci, [vp, i64]),
            "ixh_cache_contains": (ci, [vp, i64]),
            "ixh_cache_can_add": (ci, [vp]),
            "ixh_cache_block_row": (ci, [vp, i64, ci, i32p, ci]),
            "ixh_cache_slot_index": (i64, [vp, i64, ci, i64]),
            "ixh_cache_pool_stats": (None, [vp, ci, i32p, i32p]),
            "ixh_cache_check": (ci, [vp]),
            "ixh_build_batch": (ci, [vp, ci, i64p, i32p, i32p, i32p, i32p] + [i32p] * 9 + [ctypes.POINTER(ci)]),
            "ixh_cache_num_live": (ci, [vp]),
            "ixh_cache_live": (ci, [vp, i64p, ci]),
            "ixh_sched_create": (vp, [vp, ci, i64, i64]),
            "ixh_sched_destroy": (None, [vp]),
            "ixh_sched_error": (ctypes.c_char_p, [vp]),
            "ixh_sched_add": (ci, [vp, i64, i32p, ci, i64, i64, i32p, ci]),
            "ixh_sched_cancel": (None, [vp, i64]),
            "ixh_sched_has_work": (ci, [vp]),
            "ixh_sched_preemptions": (i64, [vp]),
            "ixh_sched_prepare": (ci, [vp]),
            "ixh_sched_plan_tokens": (i64, [vp]),
            "ixh_sched_plan": (None, [vp, i64p, i64p, i32p, i32p, i32p]),
            "ixh_sched_commit": (ci, [vp, i32p, ci]),
            "ixh_sched_launched": (ci, [vp]),
            "ixh_sched_resolve": (ci, [vp, i32p, ci]),
            "ixh_sched_is_planned": (ci, [vp]),
            "ixh_sched_abandon": (None, [vp]),
            "ixh_sched_plan_token_values": (None, [vp, i32p]),
            "ixh_sched_num_completed": (ci, [vp]),
            "ixh_sched_completed": (None, [vp, ci, i64p, i32p, i32p]),
            "ixh_sched_completed_tokens": (None, [vp, ci, i32p]),
            "ixh_sched_clear_completed": (None, [vp]),
            "ixh_sched_list": (ci, [vp, ci, i64p, ci]),
            "ixh_sched_seq_info": (ci, [vp, i64, i32p, i64p, i64p]),
            "ixh_sched_seq_tokens": (ci, [vp, i64, i64, i32p, i64]),
            "ixh_pool_create": (vp, [ci]),
            "ixh_pool_destroy": (None, [vp]),
            "ixh_pool_allocate": (ci, [vp]),
            "ixh_pool_release": (ci, [vp, ci]),
            "ixh_pool_free_pages": (ci, [vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _configured = True
    return lib


class PagePool:
    """A pool on its own."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._lib = host_lib()
        self._h = self._lib.ixh_pool_create(num_pages)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ixh_pool_destroy(self._h)
            self._h = None

    @property
    def free_pages(self) -> int:
        return self._lib.ixh_pool_free_pages(self._h)

    @property
    def used_pages(self) -> int:
        return self.num_pages - self.free_pages

    def allocate(self) -> Optional[int]:
        page = self._lib.ixh_pool_allocate(self._h)
        return None if page < 0 else page

    def release(self, page: int) -> None:
        rc = self._lib.ixh_pool_release(self._h, int(page))
        if rc == -1:
            raise CacheError(f"page {page} is outside the pool of {self.num_pages}")
        if rc == -2:
            raise CacheError(f"page {page} freed twice")


@dataclass(frozen=True)
class GroupLayout:
    """One page group: `window` 0 keeps every token, W > 0 only the last W.  `release_passed` False keeps the
    pages that the window has passed until the request ends (what the reference does for its windowed layers,
    src/model/gpt_oss.cc:259-262); the attention kernels mask by the window either way, so the two settings must
    give the same logits, which is what the switch is for."""

    window: int = 0
    release_passed: bool = True

    @property
    def release_window(self) -> int:
        """The window as the bookkeeping sees it: 0 if no page is ever given back early."""
        return self.window if self.release_passed else 0


class _PoolView:
    """What the manager shows of one group's pool."""

    def __init__(self, manager: "CacheManager", group: int):
        self._m, self._g = manager, group

    def _stats(self):
        num, free = ctypes.c_int32(), ctypes.c_int32()
        self._m._lib.ixh_cache_pool_stats(self._m._h, self._g, ctypes.byref(num), ctypes.byref(free))
        return num.value, free.value

    @property
    def num_pages(self) -> int:
        return self._stats()[0]

    @property
    def free_pages(self) -> int:
        return self._stats()[1]

    @property
    def used_pages(self) -> int:
        num, free = self._stats()
        return num - free


RESERVE_OK, RESERVE_POOL_EMPTY, RESERVE_CONTEXT_FULL = "ok", "pool_empty", "context_full"
_RESERVE = {0: RESERVE_OK, 1: RESERVE_POOL_EMPTY, 2: RESERVE_CONTEXT_FULL}


def pages_for_window(window: int, page_size: int, max_requests: int, max_step_tokens: int) -> int:
    """Pages that a windowed group can ever hold at once when no step brings more than `max_step_tokens` tokens
    of a request: per request the pages that cover the window behind its next position and the step in front of
    it (plus the two that the ends may straddle), for every request slot.  A pool of this size never runs out."""
    return max_requests * (-(-(window + max_step_tokens) // page_size) + 2)


class CacheManager:
    """`max_step_tokens`: the most tokens of one request that a step will ever bring, if the caller can promise one
    (a scheduler's token budget).  With it, a windowed group that gives passed pages back takes a request's pages as
    the steps reach them instead of at reservation, so its pool may be as small as `pages_for_window` says however
    long the prompts are; a step that brings more is refused.  Without it every group holds what is reserved."""

    def __init__(self, groups: Sequence[GroupLayout], pages_per_group: Sequence[int], page_size: int,
                 max_requests: int, max_seq_len: int, max_step_tokens: Optional[int] = None):
        if page_size <= 0 or max_requests <= 0 or max_seq_len <= 0:
            raise CacheError("page_size, max_requests and max_seq_len must be positive")
        if max_step_tokens is not None and max_step_tokens <= 0:
            raise CacheError("max_step_tokens must be positive")
        if len(groups) != len(pages_per_group):
            raise CacheError("one page count per group is needed")
        if any(n <= 0 for n in pages_per_group):
            raise CacheError("a page pool needs at least one page")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_requests = max_requests
        self.max_seq_len = max_seq_len
        self.max_blocks = -(-max_seq_len // page_size)
        self._lib = host_lib()
        G = len(self.groups)
        windows = (ctypes.c_int32 * max(G, 1))(*[g.release_window for g in self.groups])
        pages = (ctypes.c_int32 * max(G, 1))(*pages_per_group)
        self.max_step_tokens = max_step_tokens
        self._h = self._lib.ixh_cache_create(G, windows, pages, page_size, max_requests, max_seq_len,
                                             int(max_step_tokens or 0))
        if not self._h:
            raise CacheError("the cache manager could not be created")
        self.pools = [_PoolView(self, g) for g in range(G)]
        self._ids: Dict[Hashable, int] = {}  # request id (any hashable) -> the integer the library knows it by
        self._names: Dict[int, Hashable] = {}  # and back
        self._pinned = set()  # names that stay known while the request holds nothing (see intern)
        self._next = 0

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.ixh_cache_destroy(self._h)
            self._h = None

    def _err(self, rid=None) -> CacheError:
        msg = self._lib.ixh_cache_error(self._h).decode("utf-8", "replace")
        return CacheError(f"request {rid!r}: {msg}" if rid is not None else msg)

    def _id(self, rid) -> int:
        try:
            return self._ids[rid]
        except KeyError:
            raise CacheError(f"unknown request {rid!r}") from None

    def intern(self, rid) -> int:
        """The integer the library knows `rid` by, given out now if it has none.  A name interned here stays
        known until `forget`, also while the request holds nothing (the scheduler's library adds and frees
        requests by these integers on its own)."""
        if rid not in self._ids:
            self._ids[rid] = self._next
            self._names[self._next] = rid
            self._next += 1
        self._pinned.add(rid)
        return self._ids[rid]

    def forget(self, rid) -> None:
        self._pinned.discard(rid)
        if rid in self._ids and not self._lib.ixh_cache_contains(self._h, self._ids[rid]):
            del self._names[self._ids.pop(rid)]

    def name_of(self, ident: int):
        return self._names[ident]

    # ---- requests -------------------------------------------------------
    def __contains__(self, rid) -> bool:
        return rid in self._ids and bool(self._lib.ixh_cache_contains(self._h, self._ids[rid]))

    def live_requests(self):
        n = self._lib.ixh_cache_num_live(self._h)
        buf = (ctypes.c_int64 * max(n, 1))()
        self._lib.ixh_cache_live(self._h, buf, n)
        return [self._names[i] for i in buf[:n]]

    def can_add(self) -> bool:
        return bool(self._lib.ixh_cache_can_add(self._h))

    def add(self, rid) -> int:
        """Start a request: takes a state slot, no pages yet.  Returns the slot."""
        if rid in self:
            raise CacheError(f"request {rid!r} is already live")
        fresh = rid not in self._ids
        if fresh:
            self._ids[rid] = self._next
            self._names[self._next] = rid
            self._next += 1
        slot = self._lib.ixh_cache_add(self._h, self._ids[rid])
        if slot < 0:
            err = self._err(rid)
            if fresh:
                del self._names[self._ids.pop(rid)]
            raise err
        return slot

    def free(self, rid) -> None:
        """End a request: every page and the state slot go back."""
        if self._lib.ixh_cache_free(self._h, self._id(rid)) != 0:
            raise self._err(rid)
        if rid not in self._pinned:
            del self._names[self._ids.pop(rid)]

    def reset(self, rid) -> None:
        """Preemption by recomputation: pages go back, the request starts over at
        position 0 and keeps its slot (reference: Preempt, scheduler.cc:206-229)."""
        if self._lib.ixh_cache_reset(self._h, self._id(rid)) != 0:
            raise self._err(rid)

    # ---- pages ----------------------------------------------------------
    def cached(self, rid) -> int:
        return self._lib.ixh_cache_cached(self._h, self._id(rid))

    def slot_of(self, rid) -> int:
        return self._lib.ixh_cache_slot(self._h, self._id(rid))

    def reserve(self, rid, new_len: int) -> str:
        """Make sure pages exist for tokens [0, new_len) (as far as each group's
        window still needs them).  All groups or nothing."""
        rc = self._lib.ixh_cache_reserve(self._h, self._id(rid), int(new_len))
        if rc < 0:
            raise self._err(rid)
        return _RESERVE[rc]

    def commit(self, rid, tokens: int) -> None:
        """`tokens` more tokens are now in the cache."""
        if self._lib.ixh_cache_commit(self._h, self._id(rid), int(tokens)) != 0:
            raise self._err(rid)

    def block_row(self, rid, group: int) -> List[int]:
        """The request's pages in this group by logical page number, -1 where none is held."""
        buf = (ctypes.c_int32 * self.max_blocks)()
        n = self._lib.ixh_cache_block_row(self._h, self._id(rid), group, buf, self.max_blocks)
        if n < 0:
            raise self._err(rid)
        return list(buf[:n])

    def slot_index(self, rid, group: int, position: int) -> int:
        """Flat index page * page_size + offset of the token at `position`."""
        idx = self._lib.ixh_cache_slot_index(self._h, self._id(rid), group, int(position))
        if idx < 0:
            raise self._err(rid)
        return idx

    # ---- invariants (used by tests and by debug runs) ---------------------
    def check(self) -> None:
        """Every page is free or held exactly once; every slot likewise."""
        if self._lib.ixh_cache_check(self._h) != 0:
            raise self._err()
