"""Device memory behind the cache manager: the pages of every group of layers,
and per-request state slots.

What a page holds is the mixer's business: its `cache_need()` lists the page's
tensors (`PageTensor`: name, shape per token, where the slot axis lies, dtype)
and this file allocates, per group of layers with equal needs, one tensor
[layer][page] + page shape for each of them and hands the mixer a dict by name.
(The reference's newer engine keeps one pool indexed [slot][layer][K|V],
vt-transformer/models/qwen3-0.6b/init.vt:86-117.)  Pools start zeroed: a slot
that was never written holds finite numbers, so a masked key can never bring
a NaN into a weighted sum.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..parts.base import CacheNeed, Runtime, StateNeed
from .pages import CacheManager, GroupSpec


@dataclass
class LayerCache:
    """What a mixer sees of the cache in one step."""

    tensors: Dict[str, torch.Tensor]     # by the names of its CacheNeed: [pages] + page shape, of this schedule entry
    block_table: Optional[torch.Tensor]  # int32 [entries of the step][blocks], of the entry's group
    writes: bool                         # False: the pages are another entry's, only read here
    group: int

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.tensors[name]


def group_pages(needs: List[CacheNeed], page_bytes: List[int], page_size: int, max_requests: int, max_seq_len: int,
                max_portion: int, kv_bytes: int) -> List[int]:
    """Pages per group under a budget in bytes for all of them.  A group with a window never holds more of a
    request than its window and one portion (CacheManager.max_held_pages), so it gets pages for that, for every
    request that may run, and no more; what is left of the budget goes to the groups that keep every key, which all
    hold the same tokens and so get the same number of pages: budget // (bytes of one page of each of them together),
    as the reference sizes its one pool (vt-transformer/models/qwen3-0.6b/init.vt:109-113:
    num_blocks = budget // (block_size * per_token_bytes))."""
    whole = -(-max_seq_len // page_size)
    pages = [0] * len(needs)
    left = int(kv_bytes)
    for g, need in enumerate(needs):
        if need.window > 0:
            # (what a request holds at most, and the page of head-room per running request that the scheduler keeps
            # free when it admits another)
            per_request = min(whole, -(-(need.window + max(1, max_portion)) // page_size) + 1) + 1
            pages[g] = max(1, min(max_requests * per_request, left // max(1, page_bytes[g])))
            left -= pages[g] * page_bytes[g]
    unbounded = [g for g, need in enumerate(needs) if need.window <= 0]
    if unbounded:
        per_page = sum(page_bytes[g] for g in unbounded)
        n = left // per_page if per_page else 1
        if n < 1 and per_page:
            raise ValueError(f"a cache of {kv_bytes} bytes does not hold one page of {page_size} tokens of every group "
                             f"of layers ({per_page} bytes over {len(unbounded)} group(s) that keep every key, after "
                             f"{kv_bytes - left} bytes for the groups with a window)")
        for g in unbounded:
            pages[g] = max(1, n)
    return pages


class CacheStorage:
    def __init__(self, rt: Runtime, model, page_size: int, pool_tokens: Optional[int], max_requests: int,
                 max_seq_len: int, kv_bytes: Optional[int] = None, max_portion: Optional[int] = None):
        """`pool_tokens`: how many tokens the pages of each group hold together.  Or `kv_bytes`: a budget in bytes
        for all pages, shared by the groups according to their needs (`group_pages`); `max_portion`: the most
        tokens of one request that a step brings (the scheduler's chunk size; default: a whole sequence)."""
        self.rt = rt
        self.page_size = int(page_size)
        schedule = model.schedule
        needs: List[Optional[CacheNeed]] = []
        state_needs: List[Optional[StateNeed]] = []
        for i, e in enumerate(schedule):
            mixer = model.layers[e.layer].mixer
            need = mixer.cache_need() if hasattr(mixer, "cache_need") else None
            needs.append(need)
            state_needs.append(mixer.state_need() if hasattr(mixer, "state_need") else None)
            if e.cache_from is not None:
                src = needs[e.cache_from]
                if need is None or src is None or not need.same_layout(src):
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.cache_from}: "
                                     f"their pages differ")
        # groups of entries with their own cache and equal needs
        keys: List = []
        self.group_needs: List[CacheNeed] = []
        self.entry_group: List[Optional[int]] = [None] * len(schedule)
        self.entry_index: List[Optional[int]] = [None] * len(schedule)
        members: Dict[int, int] = {}
        for i, e in enumerate(schedule):
            if e.cache_from is not None or needs[i] is None:
                continue
            k = needs[i].group_key()
            if k not in keys:
                keys.append(k)
                self.group_needs.append(needs[i])
            g = keys.index(k)
            self.entry_group[i] = g
            self.entry_index[i] = members.get(g, 0)
            members[g] = members.get(g, 0) + 1
        for i, e in enumerate(schedule):
            if e.cache_from is not None:
                self.entry_group[i] = self.entry_group[e.cache_from]
                self.entry_index[i] = self.entry_index[e.cache_from]
        # bytes of one page of every layer of a group
        self.page_bytes = [members[g] * need.bytes_per_token(rt.dtype) * self.page_size
                           for g, need in enumerate(self.group_needs)]
        if kv_bytes is not None:
            if pool_tokens is not None:
                raise ValueError("give the cache's size in tokens or in bytes, not both")
            pages = group_pages(self.group_needs, self.page_bytes, self.page_size, max_requests, max_seq_len,
                                max_portion or max_seq_len, int(kv_bytes))
        else:
            if pool_tokens is None:
                raise ValueError("the cache needs a size: pool_tokens or kv_bytes")
            pages = [max(1, -(-int(pool_tokens) // self.page_size))] * len(self.group_needs)
        self.group_pages = pages
        self.manager = CacheManager([GroupSpec(k, need.window, n) for k, need, n in zip(keys, self.group_needs, pages)],
                                    self.page_size, max_requests, max_seq_len)
        # per group and page tensor: [layer][page] + the tensor's page shape
        self.pages: List[Dict[str, torch.Tensor]] = []
        for g, need in enumerate(self.group_needs):
            self.pages.append({t.name: torch.zeros((members[g], pages[g]) + t.page_shape(self.page_size),
                                                   dtype=t.dtype or rt.dtype, device=rt.device) for t in need.tensors})
        self.writes = [e.cache_from is None for e in schedule]
        # fixed-size state per request and schedule entry (none for attention)
        self.state: List[Optional[torch.Tensor]] = []
        for need in state_needs:
            self.state.append(None if need is None else
                              torch.zeros((max_requests,) + tuple(need.shape), dtype=need.dtype, device=rt.device))

    @property
    def num_pages(self) -> int:
        """Pages of the groups that bound a request's length (those that keep every key); of the smallest group
        if every group has a window."""
        if not self.group_pages:
            return 0
        whole = [n for n, need in zip(self.group_pages, self.group_needs) if need.window <= 0]
        return min(whole) if whole else min(self.group_pages)

    @property
    def kv_bytes(self) -> int:
        """Bytes that the pages of all groups take."""
        return sum(n * b for n, b in zip(self.group_pages, self.page_bytes))

    @property
    def n_groups(self) -> int:
        return len(self.group_needs)

    def group_window(self, g: int) -> int:
        """The window of group g's layers (0: they keep every key)."""
        return int(self.group_needs[g].window)

    def layer_caches(self, block_tables: List[torch.Tensor]) -> List[Optional[LayerCache]]:
        out: List[Optional[LayerCache]] = []
        for i, g in enumerate(self.entry_group):
            if g is None:
                out.append(None)
            else:
                idx = self.entry_index[i]
                out.append(LayerCache({name: t[idx] for name, t in self.pages[g].items()}, block_tables[g],
                                      self.writes[i], g))
        return out

    def clear_state(self, slots: List[int]) -> None:
        """A new request starts from zero state."""
        if not slots or all(s is None for s in self.state):
            return
        idx = torch.tensor(slots, dtype=torch.long, device=self.rt.device)
        for s in self.state:
            if s is not None:
                s.index_fill_(0, idx, 0)
