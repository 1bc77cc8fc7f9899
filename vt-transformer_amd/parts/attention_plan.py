"""Planning of the paged attention kernels' work for one step, on the host.

The attention mixer owns this: which of a step's entries go to which bfloat16
kernel, how their rows are cut into items, and where an item's keys are cut
into ranges whose partial results a second kernel merges.  The step function
knows nothing of it: a mixer hands the arrays it wants on the device to the
step through `prepare_step` (they travel in the step's one copy), and finds
them again in `ctx.extra` when it runs.

The reference has no counterpart: its attention is a chain of launches over a
padded [B, NH, T, F] score tensor (v1/models/qwen2-7b/inference_fp16.dag:307-318).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import numpy as np
import torch

from ..kernels.ops import ATTN_CITEM_INTS, ATTN_ITEM_INTS


@dataclass
class AttentionPlan:
    """Device views of a step's work items for one (group, window, kv heads, head size), and their workspaces."""

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
# The kernel that loads straight into LDS (head size 128), fitted to launches of 4 to 8,192 blocks (one to eight
# prompts of 256 to 4,096 tokens with up to 7,168 earlier ones, 12 to 64 query heads on 2 to 8 kv heads; the choice
# it makes is within 5 % of the best of one and two row tiles with and without cuts on each of them): a block's
# step of 64 keys takes DIRECT_STEP_US with one and two row tiles per wave, a block DIRECT_BLOCK_US beside its
# steps (until its first keys are in LDS, and its results written), DIRECT_SLOTS blocks run at a time, and a merge
# launch costs DIRECT_MERGE_US[0] + [1] per 16-row tile.
DIRECT_STEP_US = {1: 1.3, 2: 2.0}
DIRECT_START_US = 4.0
DIRECT_BLOCK_US = 4.0
DIRECT_SLOTS = 448
DIRECT_MERGE_US = (8.0, 0.03)
# ... and the cuts it is asked about: none, at TILE_CUT, and a finer one.  The finer one is for portions behind a long
# context on few kv heads, whose items are few and long (2,048 tokens behind 30,720 on 12 / 2 heads: 192 blocks of 500
# steps): two ranges each still leave a quarter of the slots empty, four fill them (476 -> 427 us; behind 14,336:
# 246 -> 226).  Measured over 39 shapes (512 to 16,384 tokens, up to 30,720 earlier ones, 12 / 2, 28 / 4 and 64 / 8
# heads, one to sixteen prompts): the model's choice among these is 1.0 % behind the best of the twelve on average
# (1.4 % without the finer cut), at worst 4 us on a 29 us launch.
DIRECT_CUTS = (0., 0.8, TILE_CUT)
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
                    split: Optional[float] = None, direct: bool = False) -> Tuple[np.ndarray, int, np.ndarray, int]:
    """Items of the LDS-tiled kernel: 64 * rt rows of one entry and the keys they may see, longest first so that
    the blocks that finish last start first.  Returns (items [n, 8], rt, combine items [m, 6], partial indices).

    `slots` blocks run at a time and the others follow as blocks finish, so a launch lasts as long as its longest
    item or as all items' steps shared out over the slots, whichever is more.  The longest items of a fresh prompt
    (its last rows see every key) are what a launch waits for when the items are few (few kv heads, one prompt):
    their keys are cut into ranges, each an item of its own, whose partial results the merge kernel adds up.
    `rt` (row tiles per wave) and `split` (the length to cut to, in units of the balanced launch; 0: no cuts)
    override the choice.

    `direct`: the kernel brings its key/value blocks from the pages straight into LDS (head size 128).  Then one and
    two row tiles, each with every cut of DIRECT_CUTS (no cut among them), are priced with a model of the launch (DIRECT_*) and the
    cheapest is taken.  Otherwise: two row tiles with cuts up to a head size of 128 (a block's step takes about as
    long with two row tiles as with one there, TILE_STEP_US), whole items and the cheaper row tiles above."""
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

    def parts_of(steps, split_: float):
        if split_ <= 0:
            return np.ones_like(steps)
        balanced = float(steps.sum()) * n_kv / slots
        target = max(TILE_MIN_STEPS, int(np.ceil(balanced * split_)))
        return np.minimum(np.where(steps > target, -(-steps // target), 1), TILE_MAX_PARTS)

    def estimate(it, rt_: int) -> float:
        steps = steps_of(it)
        return max(float(steps.max()), float(steps.sum()) * n_kv / slots) * TILE_STEP_US[rt_]

    def direct_estimate(it, rt_: int, parts) -> float:
        steps = steps_of(it)
        longest = float((-(-steps // parts)).max())
        blocks = float(parts.sum()) * n_kv
        merges = float(np.minimum(4 * rt_, -(-(it["rows"] - it["row0"]) // 16))[parts > 1].sum())
        launch = max(longest * DIRECT_STEP_US[rt_] + DIRECT_START_US,
                     (float(steps.sum()) * n_kv * DIRECT_STEP_US[rt_] + blocks * DIRECT_BLOCK_US) / DIRECT_SLOTS)
        return launch + (DIRECT_MERGE_US[0] + DIRECT_MERGE_US[1] * merges if merges else 0.)

    if direct and head_dim <= 128 and (rt is None or split is None):
        best = None
        for rt_ in ((1, 2) if rt is None else (rt,)):
            it = items_for(rt_)
            if it is None:
                return none
            for split_ in (DIRECT_CUTS if split is None else (split,)):
                cost = direct_estimate(it, rt_, parts_of(steps_of(it), split_))
                if best is None or cost < best[0]:
                    best = (cost, rt_, split_)
        _, rt, split = best
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
    parts = parts_of(steps, split)
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


DECODE_BLOCKS = 768          # blocks that a decoding launch is cut for: three to a compute unit
DECODE_BLOCKS_DIRECT = 512   # ... two where the kernel's waves load straight into two LDS buffers each (head size 128)


def decode_chunk(kv_lens: np.ndarray, p_max: int, n_kv: int = 4, want_blocks: int = DECODE_BLOCKS, min_chunk: int = 64) -> int:
    """Keys per attention item of a decoding step.  A block of four waves takes one item of one (entry, kv head);
    with enough entries every entry is one item, otherwise the keys are cut so that about `want_blocks` blocks
    run (as many as the GPU holds at a time: measured inside whole decoding steps, where the keys come from
    memory), never into more than p_max items; a multiple of 64 (the four waves take 16 keys each in turn)."""
    pairs = max(1, len(kv_lens) * n_kv)
    splits = min(p_max, max(1, -(-want_blocks // pairs)))
    longest = int(kv_lens.max())
    chunk = max(min_chunk, -(-longest // splits))
    return -(-chunk // 64) * 64


DECODE_MAX_PARTS = 16   # items that one decoding entry's keys are cut into at most


def decode_parts_max(n_positions: int) -> int:
    """The most items one entry's keys are cut into in a decoding step of an engine set up for this many positions."""
    return max(1, min(DECODE_MAX_PARTS, -(-int(n_positions) // 64)))


@dataclass
class HostPlan:
    """What the planner made on the host for one step: the arrays that go to the device, and the numbers that the
    launches need."""

    arrays: Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]   # items, combine items, tile items, their combines
    row_tiles: int
    n_parts: int
    tile_rt: int
    n_tile_parts: int

    def flat(self) -> np.ndarray:
        return np.concatenate([x.reshape(-1) for x in self.arrays]) if any(x.size for x in self.arrays) \
            else np.zeros(0, np.int32)


def plan_step(entry_start: np.ndarray, entry_pos0: np.ndarray, group: int, window: int, n_kv: int,
              head_dim: int, direct: bool = False) -> HostPlan:
    """All of a step's attention work for one kind of attention layer.  `direct`: the tiled kernel of this head
    size loads its keys and values straight into LDS (plan_tile_items)."""
    short, long = split_entries(entry_start, group)
    # (heads above 128: two row tiles per wave do not fit the registers)
    row_tiles = choose_row_tiles(entry_start, group, n_kv, short) if len(short) and head_dim <= 128 else 1
    items, citems, n_parts = plan_attention_items(entry_start, entry_pos0, group, window, n_kv, rt=row_tiles,
                                                  entries=short)
    # (heads above 128: one block per compute unit at a time)
    t_items, tile_rt, t_citems, t_parts = plan_tile_items(
        entry_start, entry_pos0, group, window, n_kv, long,
        slots=TILE_SLOTS if head_dim <= 128 else TILE_SLOTS // 2, head_dim=head_dim, direct=direct)
    return HostPlan((items, citems, t_items, t_citems), row_tiles, n_parts, tile_rt, t_parts)


def device_plan(host: HostPlan, dev: torch.Tensor, rt, n_kv: int, head_dim: int) -> AttentionPlan:
    """The plan whose arrays lie in `dev` (int32, host.flat() copied there); workspaces from the runtime."""
    lists = host.arrays
    ends = np.cumsum([x.size for x in lists])
    d_items, d_citems, d_tiles, d_tcitems = (dev[e - x.size:e] if x.size else None for x, e in zip(lists, ends))
    if d_items is None:
        d_items = dev[:0]
    part_o = part_ml = t_part_o = t_part_ml = None
    n_parts, row_tiles, t_parts, tile_rt = host.n_parts, host.row_tiles, host.n_tile_parts, host.tile_rt
    if n_parts:
        part_o = rt.buffer("attn.part_o", (n_parts * row_tiles * n_kv * 16 * head_dim,), torch.float32)
        part_ml = rt.buffer("attn.part_ml", (n_parts * row_tiles * n_kv * 16 * 2,), torch.float32)
    if t_parts:
        t_part_o = rt.buffer("attn.tile_part_o", (t_parts * 4 * tile_rt * n_kv * 16 * head_dim,), torch.float32)
        t_part_ml = rt.buffer("attn.tile_part_ml", (t_parts * 4 * tile_rt * n_kv * 16 * 2,), torch.float32)
    items, citems, t_items, t_citems = lists
    return AttentionPlan(d_items, items.shape[0], d_citems, citems.shape[0], part_o, part_ml, n_parts, row_tiles,
                         d_tiles, t_items.shape[0], tile_rt, d_tcitems, t_citems.shape[0], t_part_o, t_part_ml, t_parts)
