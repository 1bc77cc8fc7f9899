"""Device memory behind the cache manager: key and value pages per group of
layers, and per-request state slots.

Pages of a group: K [layer][page][kv head][slot][D], V [layer][page][kv head][D][slot]
(the reference's newer engine keeps one pool indexed [slot][layer][K|V],
vt-transformer/models/qwen3-0.6b/init.vt:86-117; here a page of one kv head is
contiguous so that one read of it serves all query heads of its group).
Pools start zeroed: a slot that was never written holds finite numbers, so a
masked key can never bring a NaN into a weighted sum.
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

    k: Optional[torch.Tensor]            # [pages][kv heads][slot][D] of this schedule entry
    v: Optional[torch.Tensor]            # [pages][kv heads][D][slot]
    block_table: Optional[torch.Tensor]  # int32 [entries of the step][blocks], of the entry's group
    writes: bool                         # False: the pages are another entry's, only read here
    group: int


class CacheStorage:
    def __init__(self, rt: Runtime, model, page_size: int, pool_tokens: Optional[int], max_requests: int,
                 max_seq_len: int, kv_bytes: Optional[int] = None):
        """`pool_tokens`: how many tokens the pages of each group hold together.  Or `kv_bytes`: a budget in bytes
        for all keys and values, shared by the groups: a token takes a slot of a page in every group, so every
        group gets the same number of pages, budget // (bytes of one page of each group together), as the
        reference sizes its one pool (vt-transformer/models/qwen3-0.6b/init.vt:109-113:
        num_blocks = budget // (block_size * per_token_bytes))."""
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
                if need is None or src is None or (need.kv_heads, need.head_dim) != (src.kv_heads, src.head_dim):
                    raise ValueError(f"schedule entry {i} cannot read the cache of entry {e.cache_from}: "
                                     f"their key/value heads differ")
        # groups of entries with their own cache and equal needs
        keys: List = []
        self.entry_group: List[Optional[int]] = [None] * len(schedule)
        self.entry_index: List[Optional[int]] = [None] * len(schedule)
        members: Dict[int, int] = {}
        for i, e in enumerate(schedule):
            if e.cache_from is not None or needs[i] is None:
                continue
            k = needs[i].group_key()
            if k not in keys:
                keys.append(k)
            g = keys.index(k)
            self.entry_group[i] = g
            self.entry_index[i] = members.get(g, 0)
            members[g] = members.get(g, 0) + 1
        for i, e in enumerate(schedule):
            if e.cache_from is not None:
                self.entry_group[i] = self.entry_group[e.cache_from]
                self.entry_index[i] = self.entry_index[e.cache_from]
        self.group_needs = [CacheNeed(*k) for k in keys]
        elem = torch.empty((), dtype=rt.dtype).element_size()
        # bytes of one page of every layer of a group: keys and values
        self.page_bytes = [2 * members[g] * need.kv_heads * need.head_dim * self.page_size * elem
                           for g, need in enumerate(self.group_needs)]
        if kv_bytes is not None:
            if pool_tokens is not None:
                raise ValueError("give the cache's size in tokens or in bytes, not both")
            per_page = sum(self.page_bytes)
            num_pages = int(kv_bytes) // per_page if per_page else 1
            if num_pages < 1 and per_page:
                raise ValueError(f"a cache of {kv_bytes} bytes does not hold one page of {self.page_size} tokens "
                                 f"({per_page} bytes over {len(keys)} group(s) of layers)")
            num_pages = max(1, num_pages)
        else:
            if pool_tokens is None:
                raise ValueError("the cache needs a size: pool_tokens or kv_bytes")
            num_pages = max(1, -(-int(pool_tokens) // self.page_size))
        self.num_pages = num_pages
        self.manager = CacheManager([GroupSpec(k, k[2], num_pages) for k in keys], self.page_size, max_requests,
                                    max_seq_len)
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        for g, need in enumerate(self.group_needs):
            shape_k = (members[g], num_pages, need.kv_heads, self.page_size, need.head_dim)
            shape_v = (members[g], num_pages, need.kv_heads, need.head_dim, self.page_size)
            self.k.append(torch.zeros(shape_k, dtype=rt.dtype, device=rt.device))
            self.v.append(torch.zeros(shape_v, dtype=rt.dtype, device=rt.device))
        self.writes = [e.cache_from is None for e in schedule]
        # fixed-size state per request and schedule entry (none for attention)
        self.state: List[Optional[torch.Tensor]] = []
        for need in state_needs:
            self.state.append(None if need is None else
                              torch.zeros((max_requests,) + tuple(need.shape), dtype=need.dtype, device=rt.device))

    @property
    def kv_bytes(self) -> int:
        """Bytes that the pages of all groups take."""
        return self.num_pages * sum(self.page_bytes)

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
                out.append(LayerCache(self.k[g][idx], self.v[g][idx], block_tables[g], self.writes[i], g))
        return out

    def clear_state(self, slots: List[int]) -> None:
        """A new request starts from zero state."""
        if not slots or all(s is None for s in self.state):
            return
        idx = torch.tensor(slots, dtype=torch.long, device=self.rt.device)
        for s in self.state:
            if s is not None:
                s.index_fill_(0, idx, 0)
