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

import gc
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import NO_PAGE, CacheError
from ..cache.storage import CacheStorage
from ..parts.base import HostStaging, Runtime


class OutOfPages(RuntimeError):
    """The step needs more pages than are free; nothing was changed."""


@dataclass
class StepEntry:
    rid: Hashable             # a request admitted to the cache manager
    tokens: Sequence[int]     # its next tokens (>= 1)
    want: Sequence[int] = ()  # places among these tokens whose logits are wanted


class StepContext:
    """Everything the parts may read about the step, on host and device.

    Host arrays are int32 numpy views into the step's one metadata buffer; the device views lie in the same order
    in its copy on the device.  A part that wants further integers on the device (work items of its kernels,
    lengths that its launches read from memory) returns them from `prepare_step(ctx)`, which the step function
    calls once per part after the host arrays are set and before the copy: a dict key -> int32 array.  They
    travel in the same copy and are found as `ctx.extra[key]` when the part runs; `ctx.memo` is a scratch dict of
    the step for whatever the part wants to keep on the host between the two (and for parts of the same kind to
    share one plan: a key that is already in `ctx.extra_host` need not be made again).  For steps that are
    captured and replayed the size of an array may depend on the key and the number of entries only."""

    def __init__(self, rt: Runtime, n_positions: int):
        self.rt = rt
        self.n_positions = int(n_positions)   # positions are below this (size of position tables)
        self.n_tokens = 0
        self.n_entries = 0
        self.n_logit_rows = 0
        self.single_token = False             # every entry brings exactly one token (a decoding step)
        # host arrays (numpy int32)
        self.h_token_ids = self.h_positions = self.h_tok_entry = None
        self.h_entry_start = self.h_entry_pos0 = self.h_state_slots = self.h_logit_rows = None
        self.h_kv_lens = None                 # int64 per entry: tokens the request holds after this step
        self.h_block_tables: List[np.ndarray] = []
        # device views
        self.token_ids = self.positions = self.tok_entry = None
        self.entry_start = self.entry_pos0 = self.state_slots = self.logit_rows = None
        self.block_tables: List[torch.Tensor] = []
        self.fresh: List[bool] = []           # per entry: the request's first step (its state slot was just cleared)
        self.extra_host: Dict[Hashable, np.ndarray] = {}
        self.extra: Dict[Hashable, torch.Tensor] = {}
        self.memo: Dict[Hashable, object] = {}
        self.offsets: Dict[str, object] = {}  # where the pieces lie in the metadata buffer


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


# (captured steps of 256 entries are slower than launched ones: 11.3 against 10.8 ms at 7B sizes; of 192 faster, 9.7 against 10.8)
GRAPH_BATCHES = (1, 2, 4, 8, 16, 32, 64, 96, 128, 192)


class ModelRunner:
    """Owns the model, its cache and the step function."""

    def __init__(self, model, rt: Runtime, page_size: int, pool_tokens: Optional[int], max_requests: int,
                 max_seq_len: int, kv_bytes: Optional[int] = None, max_portion: Optional[int] = None):
        self.model = model
        self.rt = rt
        self.max_seq_len = int(max_seq_len)
        self.storage = CacheStorage(rt, model, page_size, pool_tokens, max_requests, max_seq_len, kv_bytes=kv_bytes,
                                    max_portion=max_portion)
        self.cache = self.storage.manager
        self.vocab_size = model.spec.vocab_size
        self.steps = 0
        self.tokens = 0
        self._staging = HostStaging(torch.int32)
        # Decoding steps of a 16-bit model are captured once per batch size and replayed, unless a mixer keeps
        # state of its own between steps (the warm-up run before a capture would advance it twice) or a part does
        # not declare that its step can be replayed.  This is decided here, once, for the whole model: one part that
        # is stateful or says nothing keeps every step of the model on the launch-by-launch path (and the engine,
        # which asks `replays()`, then never starts a step ahead of the host); the other parts lose nothing but that.
        self.decode_graphs = False
        self._graphs: Dict[int, _DecodeGraph] = {}
        self._stateless = all(s is None for s in self.storage.state)
        parts = model.parts() if hasattr(model, "parts") else None
        self._replayable = (self._stateless and parts is not None
                            and all(bool(getattr(p, "replayable", False)) for p in parts))
        # parts that plan work of their own for a step (PagedAttention does)
        known = parts if parts is not None else [getattr(layer, "mixer", None) for layer in model.layers]
        self._preparers = [p for p in known if p is not None and hasattr(p, "prepare_step")]

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

    def _prepare_parts(self, ctx: StepContext) -> Dict[Hashable, np.ndarray]:
        """Ask every part that plans work of its own for the integers it wants on the device in this step."""
        ctx.memo, ctx.extra_host = {}, {}
        for p in self._preparers:
            got = p.prepare_step(ctx)
            if got:
                for key, arr in got.items():
                    if key not in ctx.extra_host:
                        ctx.extra_host[key] = np.ascontiguousarray(arr, dtype=np.int32).reshape(-1)
        return ctx.extra_host

    def _fill_context(self, ctx: StepContext, h: dict, rows: np.ndarray, dev: Optional[torch.Tensor]) -> torch.Tensor:
        """Lay the host arrays and what the parts add to them out in one int32 buffer, copy it to the device (`dev`,
        or the runtime's buffer for step metadata if None), and point the context at the pieces.  Returns the
        device buffer."""
        ctx.n_tokens, ctx.n_entries, ctx.n_logit_rows = h["n"], h["n_entries"], len(rows)
        ctx.single_token = h["n"] == h["n_entries"]
        ctx.h_token_ids, ctx.h_positions, ctx.h_tok_entry = h["ids"], h["positions"], h["tok_entry"]
        ctx.h_entry_start, ctx.h_entry_pos0, ctx.h_state_slots = h["start"], h["pos0"], h["slots"]
        ctx.h_logit_rows, ctx.h_block_tables, ctx.fresh = rows, h["tables"], h["fresh"]
        ctx.h_kv_lens = h["kv_lens"]
        extras = self._prepare_parts(ctx)
        # (the block tables last: a patched decoding step sends what lies in front of them, and of them only what changed)
        ng, nx = len(h["tables"]), len(extras)
        parts = [ctx.h_token_ids, ctx.h_positions, ctx.h_tok_entry, ctx.h_entry_start, ctx.h_entry_pos0,
                 ctx.h_state_slots, ctx.h_logit_rows] + list(extras.values()) + [t.reshape(-1) for t in h["tables"]]
        flat = np.concatenate(parts)
        if dev is None:
            dev = self.rt.buffer("step.meta", (flat.size,), torch.int32)
        if dev.numel() != flat.size:
            raise RuntimeError("step metadata does not fit its device buffer")
        self._staging.upload(flat, dev)
        self._last_flat = flat
        views, hviews, off, offs = [], [], 0, []
        for p in parts:
            views.append(dev[off:off + p.size])
            hviews.append(flat[off:off + p.size])
            offs.append(off)
            off += p.size
        # from here on the host arrays are views of the one buffer: patching it patches them
        (ctx.h_token_ids, ctx.h_positions, ctx.h_tok_entry, ctx.h_entry_start, ctx.h_entry_pos0, ctx.h_state_slots,
         ctx.h_logit_rows) = hviews[:7]
        (ctx.token_ids, ctx.positions, ctx.tok_entry, ctx.entry_start, ctx.entry_pos0, ctx.state_slots,
         ctx.logit_rows) = views[:7]
        ctx.h_block_tables = [v.reshape(h["n_entries"], h["max_blocks"]) for v in hviews[7 + nx:]]
        ctx.block_tables = [v.view(h["n_entries"], h["max_blocks"]) for v in views[7 + nx:]]
        ctx.extra, ctx.extra_host = {}, {}
        for key, v, hv in zip(extras, views[7:7 + nx], hviews[7:7 + nx]):
            ctx.extra[key], ctx.extra_host[key] = v, hv
        ctx.offsets = dict(ids=offs[0], positions=offs[1], pos0=offs[4], tables=offs[7 + nx:],
                           lead=offs[7 + nx] if ng else flat.size)
        return dev

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        h = self._host_arrays(entries)
        ctx = StepContext(self.rt, self.max_seq_len)
        self._fill_context(ctx, h, h["rows"], None)
        return ctx

    def replays(self, n_entries: int) -> bool:
        """Whether a decoding step of this many entries goes through a captured graph."""
        return (self.decode_graphs and self._replayable and self.rt.lowp
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
            o = g.ctx.offsets["ids"]
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
                g.ctx = StepContext(self.rt, self.max_seq_len)
                g.meta = self._fill_context(g.ctx, h, all_rows, None)
                caches = self.storage.layer_caches(g.ctx.block_tables)
                # once eagerly: loads the libraries and makes every scratch buffer, so the capture allocates nothing
                self.model.forward(g.ctx, caches, self.storage.state)
                torch.cuda.synchronize()
                g.graph = torch.cuda.CUDAGraph()
                # No cyclic garbage collection while the step is recorded: it may destroy an object that owns device
                # or pinned memory, events or another recorded graph (an engine that the caller has dropped), and
                # freeing those is not allowed while a stream records.  (Entering the recording collects first.)
                gc_was_on = gc.isenabled()
                gc.disable()
                try:
                    with torch.cuda.graph(g.graph):
                        g.logits = self.model.forward(g.ctx, caches, self.storage.state)
                finally:
                    if gc_was_on:
                        gc.enable()
                self._graphs[b] = g
            else:
                self._fill_context(g.ctx, h, all_rows, g.meta)
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
        exactly its one token: patch token ids, positions, what the parts add and the block-table entries of pages
        that were added, in the host copy of the metadata, and send it.  False if anything else changed (the caller then
        builds the metadata anew)."""
        h, flat = g.h, g.flat
        n = len(entries)
        pos0 = g.ctx.h_entry_pos0           # (a view of `flat`: the positions of the last step)
        for i, (e, rp) in enumerate(zip(entries, rps)):
            if rp.length != pos0[i] + 1 or len(e.tokens) != 1 or tuple(e.want) != g.wants[i] or rp.fresh:
                return False
            t = e.tokens[0]
            if not 0 <= t < self.vocab_size:
                raise ValueError(f"token id {int(t)} is outside the vocabulary of {self.vocab_size}")
        off = g.ctx.offsets
        ids = flat[off["ids"]:off["ids"] + n]
        ids[:] = [e.tokens[0] for e in entries]
        flat[off["positions"]:off["positions"] + n] += 1
        flat[off["pos0"]:off["pos0"] + n] += 1          # (the context's host arrays are views of `flat`)
        h["kv_lens"][:n] += 1
        # what the parts add to the metadata, made anew from the advanced positions, into the same places
        old = g.ctx.extra_host
        new = self._prepare_parts(g.ctx)
        if list(new) != list(old) or any(new[k].size != old[k].size for k in new):
            return False
        for k, arr in new.items():
            old[k][:] = arr
        g.ctx.extra_host = old
        # what goes to the device: everything in front of the block tables, and of the tables the entries that changed
        # (a request takes a page every page_size steps; the tables are n entries x max_seq_len / page_size integers)
        pieces = [(flat[:off["lead"]], g.meta[:off["lead"]])]
        mb = h["max_blocks"]
        for gi in range(self.storage.n_groups):
            base = off["tables"][gi]
            lens = g.table_lens[gi]
            windowed = self.storage.group_window(gi) > 0
            for i, rp in enumerate(rps):
                t = rp.tables[gi]
                lo = hi = base + i * mb
                if windowed:                      # pages behind the window have gone: write the row anew
                    hi = lo + len(t)
                    flat[lo:hi] = t
                elif len(t) != lens[i]:
                    lo, hi = lo + lens[i], lo + len(t)
                    flat[lo:hi] = t[lens[i]:]
                lens[i] = len(t)
                if hi > lo:
                    pieces.append((flat[lo:hi], g.meta[lo:hi]))
        g.ctx.fresh = [False] * len(g.ctx.fresh)
        self._staging.upload_pieces(pieces)
        return True
