"""Bookkeeping of cache pages, block tables and per-request state slots.
Host only: nothing here touches the device.

Shaped after the reference's PageTable and CacheManager
(vt-transformer/core/vt_pages.hpp:30-134, vt_cache.hpp:187-252):
  * a pool of pages handed out last-in-first-out, lowest id first at the
    start (vt_pages.hpp:50-57, 74-82);
  * a pool of rows, one per live request (alloc_row / free_row,
    vt_pages.hpp:60-70): here the request's *state slot*, which indexes any
    per-request state of fixed size on the device;
  * allocation for a whole batch that either succeeds for every request or
    changes nothing, and that skips a page an earlier call left half full
    (vt_cache.hpp:187-252).
Differences: the block table has one entry per page, not per token; layers
with different needs (all keys, or a window of them) form groups with pools
and tables of their own; a page that a window has passed is given back at
once; and there is no prefix tree, so a finished request returns everything
(the reference keeps prefixes in a radix tree that nothing ever evicts,
vt_cache.hpp:121-166, 264-269).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

NO_PAGE = -1


class CacheError(RuntimeError):
    """Misuse of the cache manager: a page freed twice, an unknown request, ..."""


class PagePool:
    """Page ids 0..n-1, last-in-first-out."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = int(num_pages)
        self._free: List[int] = list(range(self.num_pages - 1, -1, -1))
        self._held = [False] * self.num_pages

    @property
    def available(self) -> int:
        return len(self._free)

    def alloc(self, n: int) -> Optional[List[int]]:
        """n pages, or None (and no change) if fewer are free."""
        if n < 0:
            raise CacheError(f"cannot allocate {n} pages")
        if n > len(self._free):
            return None
        out = [self._free.pop() for _ in range(n)]
        for p in out:
            self._held[p] = True
        return out

    def free(self, pages: Sequence[int]) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages:
                raise CacheError(f"page {p} is not in 0..{self.num_pages - 1}")
            if not self._held[p]:
                raise CacheError(f"page {p} is freed twice")
            self._held[p] = False
            self._free.append(p)


class SlotPool:
    """State slots 0..n-1 (the reference's table rows), last-in-first-out."""

    def __init__(self, n: int):
        if n <= 0:
            raise CacheError(f"need at least one state slot, got {n}")
        self.n = int(n)
        self._free = list(range(self.n - 1, -1, -1))
        self._held = [False] * self.n

    @property
    def available(self) -> int:
        return len(self._free)

    def alloc(self) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.pop()
        self._held[s] = True
        return s

    def free(self, s: int) -> None:
        if not 0 <= s < self.n or not self._held[s]:
            raise CacheError(f"state slot {s} is not held")
        self._held[s] = False
        self._free.append(s)


@dataclass
class GroupSpec:
    """Layers with the same need: `window` 0 keeps every key; W > 0 keeps the last W."""

    key: Hashable
    window: int
    num_pages: int


@dataclass
class RequestPages:
    """What one live request holds."""

    rid: Hashable
    slot: int
    length: int = 0                                     # tokens whose keys and values are stored
    tables: List[List[int]] = field(default_factory=list)   # per group: page id per block, NO_PAGE where none
    fresh: bool = True                                  # no step has run for it yet (its state slot is to be cleared)


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], page_size: int, max_requests: int, max_seq_len: int):
        if page_size <= 0:
            raise CacheError(f"page size must be positive, got {page_size}")
        self.page_size = int(page_size)
        self.max_seq_len = int(max_seq_len)
        self.groups = list(groups)
        self.pools = [PagePool(g.num_pages) for g in self.groups]
        self.slots = SlotPool(max_requests)
        self.requests: Dict[Hashable, RequestPages] = {}

    # -- requests ---------------------------------------------------------
    def admit(self, rid: Hashable) -> Optional[RequestPages]:
        """A state slot and empty tables for a new request; None if no slot is free."""
        if rid in self.requests:
            raise CacheError(f"request {rid!r} is already live")
        slot = self.slots.alloc()
        if slot is None:
            return None
        rp = RequestPages(rid, slot, 0, [[] for _ in self.groups])
        self.requests[rid] = rp
        return rp

    def get(self, rid: Hashable) -> RequestPages:
        try:
            return self.requests[rid]
        except KeyError:
            raise CacheError(f"request {rid!r} is not live") from None

    def release(self, rid: Hashable) -> None:
        """The request ends (finished, aborted or preempted): all it holds goes back."""
        rp = self.get(rid)
        for gi, table in enumerate(rp.tables):
            self.pools[gi].free([p for p in table if p != NO_PAGE])
        self.slots.free(rp.slot)
        del self.requests[rid]

    # -- pages ------------------------------------------------------------
    def _first_live_block(self, gi: int, length: int) -> int:
        """Blocks before this one hold only keys that no token at position >= length can see."""
        w = self.groups[gi].window
        if w <= 0:
            return 0
        return max(0, (length - w + 1)) // self.page_size

    def max_held_pages(self, gi: int, portion: int) -> int:
        """The most pages of group gi that one request can hold at a time when no step brings more than `portion`
        of its tokens: every page for a group that keeps all keys; for a group with a window, the pages of the
        window and of one portion (and one more: neither needs to start at a page's edge)."""
        ps = self.page_size
        whole = -(-self.max_seq_len // ps)
        w = self.groups[gi].window
        if w <= 0:
            return whole
        return min(whole, -(-(w + max(1, int(portion))) // ps) + 1)

    def pages_needed(self, rp: RequestPages, new_len: int, portion: Optional[int] = None) -> List[int]:
        """Per group, how many pages `reserve` would have to take for the request to hold new_len tokens after
        one step.  With `portion` (the most tokens that a step brings): how many more pages the request will ever
        hold at a time on its way to new_len in steps of at most that many tokens, which for a group with a window
        is bounded by the window (`max_held_pages`), since `commit` gives back what the window has passed."""
        ps = self.page_size
        out = []
        for gi, table in enumerate(rp.tables):
            first = rp.length // ps
            last = (new_len + ps - 1) // ps
            n = 0
            for b in range(first, last):
                if b >= len(table) or table[b] == NO_PAGE:
                    n += 1
            if portion is not None and self.groups[gi].window > 0:
                held = sum(1 for p in table if p != NO_PAGE)
                n = min(n, max(0, self.max_held_pages(gi, portion) - held))
            out.append(n)
        return out

    def reserve(self, items: Sequence[Tuple[Hashable, int]]) -> bool:
        """Pages for every (request, new length) of a step: all of them, or none and False."""
        ps = self.page_size
        plans = []
        need = [0] * len(self.groups)
        seen = set()
        for rid, new_len in items:
            rp = self.get(rid)
            if rid in seen:
                raise CacheError(f"request {rid!r} appears twice in one step")
            seen.add(rid)
            if new_len < rp.length:
                raise CacheError(f"request {rid!r} holds {rp.length} tokens, cannot shrink to {new_len}")
            if new_len > self.max_seq_len:
                raise CacheError(f"request {rid!r} would hold {new_len} tokens, the limit is {self.max_seq_len}")
            per_group = self.pages_needed(rp, new_len)
            for gi, n in enumerate(per_group):
                need[gi] += n
            plans.append((rp, new_len))
        for gi, n in enumerate(need):
            if n > self.pools[gi].available:
                return False
        for rp, new_len in plans:
            first = rp.length // ps
            last = (new_len + ps - 1) // ps
            for gi, table in enumerate(rp.tables):
                while len(table) < last:
                    table.append(NO_PAGE)
                for b in range(first, last):
                    if table[b] == NO_PAGE:
                        table[b] = self.pools[gi].alloc(1)[0]
        return True

    def commit(self, rid: Hashable, new_len: int) -> None:
        """The step has stored keys and values up to new_len: pages that a window has passed go back."""
        rp = self.get(rid)
        if new_len < rp.length:
            raise CacheError(f"request {rid!r}: commit to {new_len} below its length {rp.length}")
        rp.length = new_len
        rp.fresh = False
        for gi, table in enumerate(rp.tables):
            dead_before = min(self._first_live_block(gi, new_len), len(table))
            gone = [table[b] for b in range(dead_before) if table[b] != NO_PAGE]
            if gone:
                self.pools[gi].free(gone)
                for b in range(dead_before):
                    table[b] = NO_PAGE

    # -- queries ----------------------------------------------------------
    def available_pages(self) -> List[int]:
        return [p.available for p in self.pools]

    def available_tokens(self) -> int:
        """Tokens that still fit, in the reference's unit (pages x page size, vt_cache.hpp:54-57),
        for the group with the fewest free pages."""
        if not self.pools:
            return self.max_seq_len * self.slots.n     # no layer keeps pages: nothing to run out of
        return min(p.available for p in self.pools) * self.page_size

    def held_pages(self) -> List[int]:
        return [sum(1 for rp in self.requests.values() for p in rp.tables[gi] if p != NO_PAGE)
                for gi in range(len(self.groups))]

    def check(self) -> None:
        """Invariants: no page lost, none held twice."""
        for gi, pool in enumerate(self.pools):
            held = [p for rp in self.requests.values() for p in rp.tables[gi] if p != NO_PAGE]
            if len(held) != len(set(held)):
                raise CacheError(f"group {gi}: a page is held twice")
            if len(held) + pool.available != pool.num_pages:
                raise CacheError(f"group {gi}: {pool.num_pages - len(held) - pool.available} pages are lost")
            for p in held:
                if not pool._held[p]:
                    raise CacheError(f"group {gi}: page {p} is in a table but marked free")
        slots = [rp.slot for rp in self.requests.values()]
        if len(slots) != len(set(slots)):
            raise CacheError("a state slot is held twice")
        if len(slots) + self.slots.available != self.slots.n:
            raise CacheError("a state slot is lost")
