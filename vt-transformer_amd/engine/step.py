"""The step function: run a batch of (request, its next tokens) from the
cache and return logits at the wanted places.

A step holds any mixture of portions of prompts and single decoded tokens,
as one flat list of tokens without padding.  The reference's step
(EngineBase::forward, vt-transformer/core/vt_engine.hpp:34-37, 66) takes a
batch that is all-prefill or all-decode (:16-22) and returns one sampled
token per request; its older engine pads a rectangular [B, T] block
(v1/tensortype/nn_kvcache.cpp:346-420).  Here positions are
start + i as there (nn_kvcache.cpp:444-448), logits come back instead of
tokens, and sampling sits above.

Per step the host builds, in one int32 buffer that goes to the device in one
copy: token ids, positions, the entry of each token, entry starts, state
slots, the rows whose logits are wanted, and one block table per group of
layers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import NO_PAGE, CacheError
from ..cache.storage import CacheStorage
from ..kernels.ops import ATTN_CITEM_INTS, ATTN_ITEM_INTS
from ..parts.base import HostStaging, Runtime


class OutOfPages(RuntimeError):
    """The step needs more pages than are free; nothing was changed."""


@dataclass
class StepEntry:
    rid: Hashable             # a request admitted to the cache manager
    tokens: Sequence[int]     # its next tokens (>= 1)
    want: Sequence[int] = ()  # places among these tokens whose logits are wanted


@dataclass
class AttentionPlan:
    items: torch.Tensor
    n_items: int
    citems: Optional[torch.Tensor]
    n_citems: int
    part_o: Optional[torch.Tensor]
    part_ml: Optional[torch.Tensor]
    n_parts: int
    rt: int = 1
    tile_items: Optional[torch.Tensor] = None     # long entries: items of the LDS-tiled kernel
    n_tile_items: int = 0
    tile_rt: int = 1
    tile_citems: Optional[torch.Tensor] = None    # ... and the merges of those whose keys were cut into ranges
    n_tile_citems: int = 0
    tile_part_o: Optional[torch.Tensor] = None
    tile_part_ml: Optional[torch.Tensor] = None
    n_tile_parts: int = 0


MAX_PARTS = 128     # the merge kernel holds the weights of at most this many items per row tile


# the tiled kernel: blocks that run at a time (two per compute unit), and microseconds per step of 64 keys of a block
# with one and two row tiles per wave (measured on 512 to 4,096-token portions with and without earlier keys)
TILE_SLOTS = 512
TILE_STEP_US = {1: 2.1, 2: 2.45}
# An item of the tiled kernel that is longer than TILE_CUT x the launch's balanced length (all items' steps shared
# out over the slots) has its keys cut into ranges of about that length, each an item of its own, merged afterwards.
# Measured with one and two row tiles and cuts at 0.7, 1, 1.4 and 2 (us, against no cut with the better of one and
# two row tiles): a fresh 2,048-token portion with 28 query / 4 kv heads 66 (77), with 12 / 2 heads 42 (56), 4,096
# tokens with 12 / 2 heads 96 (114); 2,048 tokens behind 2,048 earlier ones 148 (147), eight 1,024-token portions 102
# (102), 64 / 8 heads 103 (103): no shorter cut helped anywhere, and cuts at 1 and below cost up to a fifth where the
# items fill the GPU anyway.
TILE_CUT = 1.4
TILE_MIN_STEPS = 6      # no item's keys are cut into ranges of fewer steps than this
TILE_MAX_PARTS = 8      # ... or into more ranges than this
LONG_ENTRY_ROWS = 256   # entries with at least this many (token, head-of-group) rows go to the LDS-tiled kernel


def split_entries(entry_start: np.ndarray, group: int) -> Tuple[np.ndarray, np.ndarray]:
    """(short, long) entry indices: long portions of prompts have rows enough to fill blocks of 64 and more; the
    rest (decoded tokens, short portions) is cut into 16-row items whose keys may be split."""
    rows = (entry_start[1:] - entry_start[:-1]).astype(np.int64) * group
    idx = np.arange(len(rows))
    return idx[rows < LONG_ENTRY_ROWS], idx[rows >= LONG_ENTRY_ROWS]


def plan_tile_items(entry_start: np.ndarray, entry_pos0: np.ndarray, group: int, window: int, n_kv: int,
                    entries: np.ndarray, rt: Optional[int] = None, slots: int = TILE_SLOTS, head_dim: int = 128,
                    split: Optional[float] = None) -> Tuple[np.ndarray, int, np.ndarray, int]:
    """Items of the LDS-tiled kernel: 64 * rt rows of one entry and the keys they may see, longest first so that
    the blocks that finish last start first.  Returns (items [n, 8], rt, combine items [m, 6], partial indices).

    A block's step over 64 keys takes about as long with two row tiles per wave as with one (TILE_STEP_US), because
    a wave waits on its own chain of loads, products and exponentials more than on the machine; `slots` blocks run
    at a time and the others follow as blocks finish, so a launch lasts as long as its longest item or as all items'
    steps shared out over the slots, whichever is more.  The longest items of a fresh prompt (its last rows see
    every key) are what a launch waits for when the items are few (few kv heads, one prompt): their keys are cut
    into ranges, each an item of its own, whose partial results the merge kernel adds up (TILE_CUT).  `rt` (row
    tiles per wave) and `split` (the length to cut to, in units of the balanced launch; 0: no cuts) override the
    choice.  Heads above 128 keep whole items and choose rt by the estimate."""
    q_len = (entry_start[1:] - entry_start[:-1]).astype(np.int64)[entries]
    rows = q_len * group
    e_pos0_all = entry_pos0[entries].astype(np.int64)
    none = (np.zeros((0, ATTN_ITEM_INTS), np.int32), rt or 1, np.zeros((0, ATTN_CITEM_INTS), np.int32), 0)

    def items_for(rt_: int):
        rpi = 64 * rt_
        n_tiles = (rows + rpi - 1) // rpi
        total = int(n_tiles.sum())
        if total == 0:
            return None
        which = np.repeat(np.arange(len(entries)), n_tiles)
        first = np.cumsum(n_tiles) - n_tiles
        row0 = (np.arange(total) - np.repeat(first, n_tiles)) * rpi
        ent = entries[which]
        e_rows, e_len = rows[which], q_len[which]
        e_pos0, e_start = e_pos0_all[which], entry_start[:-1][ent].astype(np.int64)
        min_p = e_pos0 + row0 // group
        max_p = e_pos0 + np.minimum(e_rows - 1, row0 + rpi - 1) // group
        lo = np.maximum(0, min_p - window + 1) if window > 0 else np.zeros_like(min_p)
        return dict(ent=ent, start=e_start, len=e_len, pos0=e_pos0, row0=row0, rows=e_rows, lo=(lo // 16) * 16, hi=max_p + 1)

    def steps_of(it):
        return (it["hi"] - it["lo"] + 63) // 64

    def estimate(it, rt_: int) -> float:
        steps = steps_of(it)
        return max(float(steps.max()), float(steps.sum()) * n_kv / slots) * TILE_STEP_US[rt_]

    if rt is None:
        if head_dim <= 128:
            rt = 2          # (measured: with the longest items cut, two row tiles are as good as one or better)
        else:
            cands = [items_for(1), items_for(2)]
            if cands[0] is None:
                return none
            rt = 1 if estimate(cands[0], 1) <= estimate(cands[1], 2) else 2
    if split is None:
        split = TILE_CUT if head_dim <= 128 else 0.
    it = items_for(rt)
    if it is None:
        return none
    steps = steps_of(it)
    parts = np.ones_like(steps)
    if split > 0:
        balanced = float(steps.sum()) * n_kv / slots
        target = max(TILE_MIN_STEPS, int(np.ceil(balanced * split)))
        parts = np.minimum(np.where(steps > target, -(-steps // target), 1), TILE_MAX_PARTS)
    total = len(parts)
    n_all = int(parts.sum())
    of = np.repeat(np.arange(total), parts)                   # item that each part belongs to
    p_first = np.cumsum(parts) - parts
    j = np.arange(n_all) - np.repeat(p_first, parts)          # index of the part within its item
    per = (-(-steps // parts)) * 64                            # keys per part: whole steps
    lo = it["lo"][of] + j * per[of]
    hi = np.minimum(it["hi"][of], lo + per[of])
    multi = parts > 1
    part0 = np.cumsum(np.where(multi, parts, 0)) - np.where(multi, parts, 0)      # partial indices of split items
    part_id = np.where(multi[of], part0[of] + j, -1)
    items = np.stack([it["ent"][of], it["start"][of], it["len"][of], it["pos0"][of], it["row0"][of], lo, hi, part_id], axis=1)
    keep = hi > lo                                            # (a last part can be empty when the steps do not divide)
    order = np.argsort(-(hi - lo)[keep], kind="stable")
    items = items[keep][order].astype(np.int32)
    # an empty part still counts among its item's parts: its slot is never written, so it must not be merged.
    n_real = np.bincount(of[keep], minlength=total)
    cl = []
    m = np.nonzero(multi)[0]
    for t in range(4 * rt):
        r0 = it["row0"][m] + 16 * t
        ok = r0 < it["rows"][m]
        mm = m[ok]
        cl.append(np.stack([it["start"][mm], it["len"][mm], r0[ok], part0[mm], n_real[mm], np.full(len(mm), t)], axis=1))
    citems = np.concatenate(cl).astype(np.int32) if cl else np.zeros((0, ATTN_CITEM_INTS), np.int32)
    return items, rt, citems, int(np.where(multi, parts, 0).sum())


def choose_row_tiles(entry_start: np.ndarray, group: int, n_kv: int, entries: np.ndarray, min_items: int = 768) -> int:
    """Row tiles (of 16 rows) per item of the per-wave kernel: two if that still leaves enough items to fill the
    GPU (every key/value block read then serves twice the rows)."""
    q_len = (entry_start[1:] - entry_start[:-1]).astype(np.int64)[entries]
    items = int(((q_len * group + 31) // 32).sum()) * n_kv
    return 2 if items >= min_items else 1


def plan_attention_items(entry_start: np.ndarray, entry_pos0: np.ndarray, group: int, window: int, n_kv: int,
                         target_waves: int = 2048, min_chunk: int = 32, rt: int = 1,
                         entries: Optional[np.ndarray] = None) -> Tuple[np.ndarray, np.ndarray, int]:
    """Work items of the bf16 attention kernel for one step.

    Rows of an entry are (token, query head of a kv group) pairs, token-major.  An item is 16 * rt rows (rt row
    tiles) against the keys [key_lo, key_hi) that any of them may see.  When the items are too few to fill the
    GPU, an item's keys are cut at absolute multiples of a chunk length into several items whose partial results
    a second kernel merges, tile by tile.
    Returns (items [n, 8], combine items [m, 6], number of partial indices)."""
    if entries is None:
        entries = np.arange(len(entry_pos0))
    rpi = 16 * rt
    q_len = (entry_start[1:] - entry_start[:-1]).astype(np.int64)[entries]
    rows = q_len * group
    n_tiles = (rows + rpi - 1) // rpi
    total = int(n_tiles.sum())
    if total == 0:
        return np.zeros((0, ATTN_ITEM_INTS), np.int32), np.zeros((0, ATTN_CITEM_INTS), np.int32), 0
    which = np.repeat(np.arange(len(entries)), n_tiles)
    first = np.cumsum(n_tiles) - n_tiles
    tile_in_entry = np.arange(total) - np.repeat(first, n_tiles)
    row0 = tile_in_entry * rpi
    ent = entries[which]
    e_rows, e_len = rows[which], q_len[which]
    e_pos0, e_start = entry_pos0[ent].astype(np.int64), entry_start[:-1][ent].astype(np.int64)
    t_first = row0 // group
    t_last = np.minimum(e_rows - 1, row0 + rpi - 1) // group
    min_p, max_p = e_pos0 + t_first, e_pos0 + t_last
    lo = np.maximum(0, min_p - window + 1) if window > 0 else np.zeros_like(min_p)
    key_lo = (lo // 16) * 16
    key_hi = max_p + 1
    span = key_hi - key_lo
    # split keys only if the items alone leave most of the GPU idle
    chunk = 0
    if total * n_kv < target_waves // 2:
        keys_total = int(span.sum()) * n_kv
        chunk = max(min_chunk, -(-keys_total // target_waves), -(-int(span.max() + 15) // MAX_PARTS))
        chunk = -(-chunk // 16) * 16
        if chunk >= int(span.max()):
            chunk = 0
    if chunk == 0:
        items = np.stack([ent, e_start, e_len, e_pos0, row0, key_lo, key_hi, np.full(total, -1)], axis=1)
        return items.astype(np.int32), np.zeros((0, ATTN_CITEM_INTS), np.int32), 0
    c_first = key_lo // chunk
    c_last = (key_hi - 1) // chunk
    n_parts = (c_last - c_first + 1)
    tot_parts = int(n_parts.sum())
    tile_of = np.repeat(np.arange(total), n_parts)
    p_first = np.cumsum(n_parts) - n_parts
    c_idx = np.arange(tot_parts) - np.repeat(p_first, n_parts) + c_first[tile_of]
    p_lo = np.maximum(key_lo[tile_of], c_idx * chunk)
    p_hi = np.minimum(key_hi[tile_of], (c_idx + 1) * chunk)
    single = (n_parts == 1)[tile_of]
    part_id = np.where(single, -1, np.arange(tot_parts))
    items = np.stack([ent[tile_of], e_start[tile_of], e_len[tile_of], e_pos0[tile_of], row0[tile_of], p_lo, p_hi,
                      part_id], axis=1).astype(np.int32)
    # one merge per 16-row tile of every item whose keys were split
    multi = np.nonzero(n_parts > 1)[0]
    cl = []
    for sub in range(rt):
        r0 = row0[multi] + 16 * sub
        keep = r0 < e_rows[multi]
        m = multi[keep]
        cl.append(np.stack([e_start[m], e_len[m], r0[keep], p_first[m], n_parts[m], np.full(len(m), sub)], axis=1))
    citems = np.concatenate(cl).astype(np.int32) if cl else np.zeros((0, ATTN_CITEM_INTS), np.int32)
    return items, citems, tot_parts


class StepContext:
    """Everything the parts may read about the step, on host and device."""

    def __init__(self, rt: Runtime, n_positions: int):
        self.rt = rt
        self.n_positions = int(n_positions)   # positions are below this (size of position tables)
        self.n_tokens = 0
        self.n_entries = 0
        self.n_logit_rows = 0
        # host arrays (numpy int32)
        self.h_token_ids = self.h_positions = self.h_tok_entry = None
        self.h_entry_start = self.h_entry_pos0 = self.h_state_slots = self.h_logit_rows = None
        self.h_block_tables: List[np.ndarray] = []
        # device views
        self.token_ids = self.positions = self.tok_entry = None
        self.entry_start = self.entry_pos0 = self.state_slots = self.logit_rows = None
        self.block_tables: List[torch.Tensor] = []
        self.fresh: List[bool] = []           # per entry: the request's first step (its state slot was just cleared)
        # set when every entry brings exactly one token (decoding): int32 device array of the number of keys per
        # attention item, by bucket of the number of kv heads (decode_bucket), and the number of items per entry
        self.decode_params: Optional[torch.Tensor] = None
        self.decode_p_max = 0
        self._plans: Dict[Tuple[int, int, int, int], AttentionPlan] = {}

    def attention_plan(self, group: int, window: int, n_kv: int, head_dim: int) -> AttentionPlan:
        key = (group, window, n_kv, head_dim)
        plan = self._plans.get(key)
        if plan is None:
            plan = self._make_plan(key)
            self._plans[key] = plan
        return plan

    def _make_plan(self, key) -> AttentionPlan:
        group, window, n_kv, head_dim = key
        short, long = split_entries(self.h_entry_start, group)
        # (heads above 128: two row tiles per wave do not fit the registers)
        row_tiles = choose_row_tiles(self.h_entry_start, group, n_kv, short) if len(short) and head_dim <= 128 else 1
        items, citems, n_parts = plan_attention_items(self.h_entry_start, self.h_entry_pos0, group, window, n_kv,
                                                      rt=row_tiles, entries=short)
        # (heads above 128: one block per compute unit at a time)
        t_items, tile_rt, t_citems, t_parts = plan_tile_items(
            self.h_entry_start, self.h_entry_pos0, group, window, n_kv, long,
            slots=TILE_SLOTS if head_dim <= 128 else TILE_SLOTS // 2, head_dim=head_dim)
        rt = self.rt
        tag = f"attnplan.{group}.{window}.{n_kv}.{head_dim}"
        lists = [items, citems, t_items, t_citems]
        flat = np.concatenate([x.reshape(-1) for x in lists])
        dev = rt.buffer(tag, (max(flat.size, 1),), torch.int32)
        if flat.size:
            dev[:flat.size].copy_(torch.from_numpy(flat))
        ends = np.cumsum([x.size for x in lists])
        d_items, d_citems, d_tiles, d_tcitems = (dev[e - x.size:e] if x.size else None for x, e in zip(lists, ends))
        if d_items is None:
            d_items = dev[:0]
        part_o = part_ml = t_part_o = t_part_ml = None
        if n_parts:
            part_o = rt.buffer("attn.part_o", (n_parts * row_tiles * n_kv * 16 * head_dim,), torch.float32)
            part_ml = rt.buffer("attn.part_ml", (n_parts * row_tiles * n_kv * 16 * 2,), torch.float32)
        if t_parts:
            t_part_o = rt.buffer("attn.tile_part_o", (t_parts * 4 * tile_rt * n_kv * 16 * head_dim,), torch.float32)
            t_part_ml = rt.buffer("attn.tile_part_ml", (t_parts * 4 * tile_rt * n_kv * 16 * 2,), torch.float32)
        return AttentionPlan(d_items, items.shape[0], d_citems, citems.shape[0], part_o, part_ml, n_parts, row_tiles,
                             d_tiles, t_items.shape[0], tile_rt, d_tcitems, t_citems.shape[0], t_part_o, t_part_ml, t_parts)


DECODE_BUCKETS = 8      # chunk lengths for 1, 2-3, 4-7, ... 128+ key/value heads


def decode_bucket(n_kv: int) -> int:
    return min(DECODE_BUCKETS - 1, max(1, int(n_kv)).bit_length() - 1)


def decode_chunk(kv_lens: np.ndarray, p_max: int, n_kv: int = 4, want_blocks: int = 768, min_chunk: int = 64) -> int:
    """Keys per attention item of a decoding step.  A block of four waves takes one item of one (entry, kv head);
    with enough entries every entry is one item, otherwise the keys are cut so that about `want_blocks` blocks
    run (three to a compute unit: measured inside whole decoding steps, where the keys come from memory), never into more than p_max items; a multiple of 64 (the four waves take 16 keys each in turn)."""
    pairs = max(1, len(kv_lens) * n_kv)
    splits = min(p_max, max(1, -(-want_blocks // pairs)))
    longest = int(kv_lens.max())
    chunk = max(min_chunk, -(-longest // splits))
    return -(-chunk // 64) * 64


class _DecodeGraph:
    """A captured decoding step for a fixed number of entries."""

    def __init__(self):
        self.graph = None
        self.ctx: Optional[StepContext] = None
        self.meta: Optional[torch.Tensor] = None
        self.logits: Optional[torch.Tensor] = None
        # what the next step through this graph needs to patch the metadata instead of building it anew
        self.rps = None             # what the requests of the last step hold (RequestPages), in order: the very
                                    # objects, since a request that ended and one admitted later may share a name
        self.h = None               # its host arrays
        self.flat = None            # its metadata as one int32 array
        self.table_lens = None      # per group and entry, the block-table entries already written
        self.wants = None
        self.wanted = None          # the view of `logits` that the last step returned


GRAPH_BATCHES = (1, 2, 4, 8, 16, 32, 64)


class ModelRunner:
    """Owns the model, its cache and the step function."""

    def __init__(self, model, rt: Runtime, page_size: int, pool_tokens: int, max_requests: int, max_seq_len: int):
        self.model = model
        self.rt = rt
        self.max_seq_len = int(max_seq_len)
        self.storage = CacheStorage(rt, model, page_size, pool_tokens, max_requests, max_seq_len)
        self.cache = self.storage.manager
        self.vocab_size = model.spec.vocab_size
        self.steps = 0
        self.tokens = 0
        self._staging = HostStaging(torch.int32)
        self.decode_p_max = max(1, min(16, -(-self.max_seq_len // 64)))   # items one entry's keys are cut into at most
        # Decoding steps of a bfloat16 model are captured once per batch size and replayed, unless a mixer keeps
        # state of its own between steps (the warm-up run before a capture would advance it twice) or a part does
        # not declare that its step can be replayed.
        self.decode_graphs = False
        self._graphs: Dict[int, _DecodeGraph] = {}
        self._stateless = all(s is None for s in self.storage.state)
        parts = model.parts() if hasattr(model, "parts") else None
        self._replayable = (self._stateless and parts is not None
                            and all(bool(getattr(p, "replayable", False)) for p in parts))

    # -- requests -----------------------------------------------------------
    def admit(self, rid: Hashable) -> bool:
        return self.cache.admit(rid) is not None

    def release(self, rid: Hashable) -> None:
        self.cache.release(rid)

    # -- the step -----------------------------------------------------------
    def _host_arrays(self, entries: Sequence[StepEntry], pad_to: int = 0, fixed_blocks: int = 0):
        cache, ps = self.cache, self.cache.page_size
        n_entries = len(entries)
        lens = np.array([len(e.tokens) for e in entries], dtype=np.int64)
        if n_entries == 0 or (lens <= 0).any():
            raise ValueError("a step needs at least one entry and every entry at least one token")
        n = int(lens.sum())
        rps = [cache.get(e.rid) for e in entries]
        pos0 = np.array([rp.length for rp in rps], dtype=np.int64)
        ids = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=n)
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            bad = ids[(ids < 0) | (ids >= self.vocab_size)][0]
            raise ValueError(f"token id {int(bad)} is outside the vocabulary of {self.vocab_size}")
        slots = np.array([rp.slot for rp in rps], dtype=np.int64)
        n_pad = max(0, pad_to - n_entries)   # padding entries: one token at position 0 with no pages
        if n_pad:
            lens = np.concatenate([lens, np.ones(n_pad, np.int64)])
            pos0 = np.concatenate([pos0, np.zeros(n_pad, np.int64)])
            ids = np.concatenate([ids, np.zeros(n_pad, np.int64)])
            slots = np.concatenate([slots, np.zeros(n_pad, np.int64)])
        n_all = n_entries + n_pad
        start = np.zeros(n_all + 1, dtype=np.int64)
        np.cumsum(lens, out=start[1:])
        tok_entry = np.repeat(np.arange(n_all), lens)
        positions = np.arange(n + n_pad) - start[:-1][tok_entry] + pos0[tok_entry]
        rows = []
        for i, e in enumerate(entries):
            for w in e.want:
                if not 0 <= w < lens[i]:
                    raise ValueError(f"request {e.rid!r}: wanted place {w} is not among its {lens[i]} tokens")
                rows.append(start[i] + w)
        new_len = pos0 + lens
        if fixed_blocks:
            max_blocks = fixed_blocks
        else:
            max_blocks = int(-(-new_len.max() // ps))
            max_blocks = -(-max_blocks // 8) * 8
        tables = []
        for gi in range(self.storage.n_groups):
            bt = np.full((n_all, max_blocks), NO_PAGE, dtype=np.int32)
            for i, rp in enumerate(rps):
                t = rp.tables[gi]
                bt[i, :len(t)] = t
            tables.append(bt)
        return dict(n=n + n_pad, n_entries=n_all, ids=ids.astype(np.int32), positions=positions.astype(np.int32),
                    tok_entry=tok_entry.astype(np.int32), start=start.astype(np.int32), pos0=pos0.astype(np.int32),
                    slots=slots.astype(np.int32), rows=np.array(rows, dtype=np.int32), tables=tables,
                    fresh=[rp.fresh for rp in rps] + [False] * n_pad, kv_lens=new_len, max_blocks=max_blocks)

    def _fill_context(self, ctx: StepContext, h: dict, rows: np.ndarray, dev: torch.Tensor, decode: bool) -> None:
        """Lay the host arrays out in one int32 buffer, copy it to `dev`, and point the context at the pieces."""
        ctx.n_tokens, ctx.n_entries, ctx.n_logit_rows = h["n"], h["n_entries"], len(rows)
        ctx.h_token_ids, ctx.h_positions, ctx.h_tok_entry = h["ids"], h["positions"], h["tok_entry"]
        ctx.h_entry_start, ctx.h_entry_pos0, ctx.h_state_slots = h["start"], h["pos0"], h["slots"]
        ctx.h_logit_rows, ctx.h_block_tables, ctx.fresh = rows, h["tables"], h["fresh"]
        dec = np.zeros(DECODE_BUCKETS, np.int32)
        if decode:
            for b in range(DECODE_BUCKETS):
                dec[b] = decode_chunk(h["kv_lens"], self.decode_p_max, n_kv=1 << b)
        parts = [ctx.h_token_ids, ctx.h_positions, ctx.h_tok_entry, ctx.h_entry_start, ctx.h_entry_pos0,
                 ctx.h_state_slots, ctx.h_logit_rows, dec] + [t.reshape(-1) for t in h["tables"]]
        flat = np.concatenate(parts)
        if dev.numel() != flat.size:
            raise RuntimeError("step metadata does not fit its device buffer")
        self._staging.upload(flat, dev)
        self._last_flat = flat
        views, off, offs = [], 0, []
        for p in parts:
            views.append(dev[off:off + p.size])
            offs.append(off)
            off += p.size
        ctx.part_offsets = dict(ids=offs[0], positions=offs[1], pos0=offs[4], dec=offs[7], tables=offs[8:])
        (ctx.token_ids, ctx.positions, ctx.tok_entry, ctx.entry_start, ctx.entry_pos0, ctx.state_slots,
         ctx.logit_rows) = views[:7]
        ctx.decode_params = views[7] if decode else None
        ctx.decode_p_max = self.decode_p_max if decode else 0
        ctx.block_tables = [v.view(h["n_entries"], h["max_blocks"]) for v in views[8:]]

    def _meta_size(self, h: dict, n_rows: int) -> int:
        return 3 * h["n"] + (h["n_entries"] + 1) + 2 * h["n_entries"] + n_rows + DECODE_BUCKETS + \
            self.storage.n_groups * h["n_entries"] * h["max_blocks"]

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        h = self._host_arrays(entries)
        decode = self.rt.dtype == torch.bfloat16 and all(len(e.tokens) == 1 for e in entries)
        ctx = StepContext(self.rt, self.max_seq_len)
        dev = self.rt.buffer("step.meta", (self._meta_size(h, len(h["rows"])),), torch.int32)
        self._fill_context(ctx, h, h["rows"], dev, decode)
        return ctx

    def replays(self, n_entries: int) -> bool:
        """Whether a decoding step of this many entries goes through a captured graph."""
        return (self.decode_graphs and self._replayable and self.rt.dtype == torch.bfloat16
                and 0 < n_entries <= GRAPH_BATCHES[-1])

    def step(self, entries: Sequence[StepEntry], ids_dev: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run the entries' tokens as one batch.  Returns fp32 logits [wanted places, vocab] on the device in the
        order of the entries and of their `want`, or None if nothing is wanted.  Raises OutOfPages (with nothing
        changed) if the cache cannot hold the new tokens.
        ids_dev (int32 on the device, one per entry): the entries' one token each, where the host does not know
        them yet (the entries then carry placeholders); only for decoding steps that `replays()` says are captured."""
        cache = self.cache
        use_graph = self.replays(len(entries)) and all(len(e.tokens) == 1 for e in entries)
        if ids_dev is not None and not use_graph:
            raise RuntimeError("token ids that are still on the device can only be fed to a captured decoding step")
        targets = [(e.rid, cache.get(e.rid).length + len(e.tokens)) for e in entries]
        for rid, new_len in targets:
            if new_len > self.max_seq_len:
                raise CacheError(f"request {rid!r} would reach {new_len} tokens, the engine is set up for {self.max_seq_len}")
        if not cache.reserve(targets):
            raise OutOfPages(f"the step needs more pages than are free ({cache.available_pages()} free per group)")
        fresh_slots = [cache.get(e.rid).slot for e in entries if cache.get(e.rid).fresh]
        self.storage.clear_state(fresh_slots)
        if use_graph:
            logits = self._step_decode_graph(entries, ids_dev)
        else:
            ctx = self.build_context(entries)
            caches = self.storage.layer_caches(ctx.block_tables)
            logits = self.model.forward(ctx, caches, self.storage.state)
        for rid, new_len in targets:
            cache.commit(rid, new_len)
        self.steps += 1
        self.tokens += sum(len(e.tokens) for e in entries)
        return logits

    # -- decoding through a captured graph ---------------------------------------
    def _feed_ids(self, g: "_DecodeGraph", ids_dev: Optional[torch.Tensor], n: int) -> None:
        """Token ids that the sampler left on the device go into the step's metadata there, after the host's copy
        of it (which holds placeholders for them) has been sent and before the step runs."""
        if ids_dev is not None:
            o = g.ctx.part_offsets["ids"]
            g.meta[o:o + n].copy_(ids_dev[:n])

    def _step_decode_graph(self, entries: Sequence[StepEntry], ids_dev: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        n = len(entries)
        b = next(x for x in GRAPH_BATCHES if x >= n)
        g = self._graphs.get(b)
        rps = [self.cache.get(e.rid) for e in entries]
        if (g is not None and g.rps is not None and len(g.rps) == n and all(a is b for a, b in zip(g.rps, rps))
                and self._advance_decode_meta(g, entries, rps)):
            self._feed_ids(g, ids_dev, n)
            g.graph.replay()        # the same requests as in the last step, one token further: the metadata was patched
            return g.wanted
        fixed_blocks = -(-self.max_seq_len // self.cache.page_size)
        h = self._host_arrays(entries, pad_to=b, fixed_blocks=fixed_blocks)
        all_rows = np.arange(b, dtype=np.int32)     # logits of every entry; the wanted ones are picked afterwards
        with self.rt.scoped(f"graph{b}:"):
            if g is None:
                g = _DecodeGraph()
                g.meta = self.rt.buffer("step.meta", (self._meta_size(h, b),), torch.int32)
                g.ctx = StepContext(self.rt, self.max_seq_len)
                self._fill_context(g.ctx, h, all_rows, g.meta, decode=True)
                caches = self.storage.layer_caches(g.ctx.block_tables)
                # once eagerly: loads the libraries and makes every scratch buffer, so the capture allocates nothing
                self.model.forward(g.ctx, caches, self.storage.state)
                torch.cuda.synchronize()
                g.graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g.graph):
                    g.logits = self.model.forward(g.ctx, caches, self.storage.state)
                self._graphs[b] = g
            else:
                self._fill_context(g.ctx, h, all_rows, g.meta, decode=True)
            self._feed_ids(g, ids_dev, n)
            g.graph.replay()
        # what the next step can patch instead of building anew: the host copy of the metadata and where its parts lie
        g.rps, g.h, g.flat = rps, h, self._last_flat
        g.table_lens = [[len(self.cache.get(e.rid).tables[gi]) for e in entries] for gi in range(self.storage.n_groups)]
        g.wants = [tuple(e.want) for e in entries]
        if len(h["rows"]) == 0:
            g.wanted = None
        elif (h["rows"] == all_rows[:len(h["rows"])]).all():
            g.wanted = g.logits[:len(h["rows"])]     # the first entries in order: a view, no copy
        else:
            g.wanted = None
            g.rps = None                             # wanted rows that are no plain prefix: no patching next time
            return g.logits.index_select(0, torch.from_numpy(h["rows"].astype(np.int64)).to(self.rt.device))
        return g.wanted

    def _advance_decode_meta(self, g: "_DecodeGraph", entries: Sequence[StepEntry], rps) -> bool:
        """The last step through this graph had the same requests in the same order, and each has since grown by
        exactly its one token: patch token ids, positions, decode chunks and the block-table entries of pages that
        were added, in the host copy of the metadata, and send it.  False if anything else changed (the caller then
        builds the metadata anew)."""
        h, flat = g.h, g.flat
        n = len(entries)
        pos0 = h["pos0"]
        for i, (e, rp) in enumerate(zip(entries, rps)):
            if rp.length != pos0[i] + 1 or len(e.tokens) != 1 or tuple(e.want) != g.wants[i] or rp.fresh:
                return False
            t = e.tokens[0]
            if not 0 <= t < self.vocab_size:
                raise ValueError(f"token id {int(t)} is outside the vocabulary of {self.vocab_size}")
        off = g.ctx.part_offsets
        ids = flat[off["ids"]:off["ids"] + n]
        ids[:] = [e.tokens[0] for e in entries]
        flat[off["positions"]:off["positions"] + n] += 1
        flat[off["pos0"]:off["pos0"] + n] += 1
        pos0[:n] += 1
        h["kv_lens"][:n] += 1
        dec = flat[off["dec"]:off["dec"] + DECODE_BUCKETS]
        for bkt in range(DECODE_BUCKETS):
            dec[bkt] = decode_chunk(h["kv_lens"], self.decode_p_max, n_kv=1 << bkt)
        mb = h["max_blocks"]
        for gi in range(self.storage.n_groups):
            base = off["tables"][gi]
            lens = g.table_lens[gi]
            windowed = self.storage.group_window(gi) > 0
            for i, rp in enumerate(rps):
                t = rp.tables[gi]
                if windowed:                      # pages behind the window have gone: write the row anew
                    row = flat[base + i * mb:base + i * mb + len(t)]
                    row[:] = t
                elif len(t) != lens[i]:
                    flat[base + i * mb + lens[i]:base + i * mb + len(t)] = t[lens[i]:]
                lens[i] = len(t)
        g.ctx.fresh = [False] * len(g.ctx.fresh)
        self._staging.upload(flat, g.meta)
        return True
