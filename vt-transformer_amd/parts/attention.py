"""Attention mixer over paged keys and values: grouped-query heads, optional
bias on the projections, optional window, position encoding as a part of its
own.

Per token, in the order of the reference's layer program
(v1/models/qwen2-7b/inference_fp16.dag:296-322): K, Q and V projections with
bias (:296, :302, :312), rotary encoding of K and Q (:297, :303), keys and
values kept for later steps (:298, :313), scores scaled by 1/sqrt(D), causal
mask, fp32 softmax, weighted sum (:307-318), output projection without bias
(:322).  The three projections are one matrix product here (rows of Q, then
K, then V), rotation is fused with the write into the cache pages, and
scores, mask, softmax and weighted sum are one kernel that reads the pages.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional

import torch

from ..config.base import PartSpec
import numpy as np

from ..kernels import ops
from .attention_plan import DECODE_BLOCKS, DECODE_BLOCKS_DIRECT, decode_chunk, decode_parts_max, device_plan, plan_step
from .base import MIXERS, POSITIONS, CacheNeed, PageTensor, Part, Runtime, StateNeed, TensorDecl
from .linear import can_add_residual, linear

# the decoding kernels take the (token, head-of-group) rows of one entry as one tile of 16
DECODE_MAX_GROUP = 16


@MIXERS.register("attention")
class PagedAttention(Part):
    takes_normed_input = True     # the q/k/v product applies the norm in front of it when the rows are few
    hands_norm_on = True          # ... and the output product prepares the norm behind it

    def adds_residual(self, rows: int) -> bool:
        """Whether the output product adds to the residual stream itself at this many rows."""
        return can_add_residual(self.rt, rows, self.width, self.nh * self.d)

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, num_kv_heads: int, head_dim: int,
                 qkv_bias: bool = False, out_bias: bool = False, window: int = 0,
                 position: Optional[PartSpec] = None, scale: Optional[float] = None, shared: Optional[dict] = None,
                 names: Optional[Dict[str, str]] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        self.rt = rt
        self.width = int(width)
        self.nh, self.nkv, self.d = int(num_heads), int(num_kv_heads), int(head_dim)
        if rt.lowp and (self.d % 16 or not 16 <= self.d <= 256):
            raise ValueError(f"head size {self.d}: the 16-bit attention kernels take multiples of 16 from 16 to 256")
        if not rt.lowp and not 1 <= self.d <= ops.ATTN_F32_MAX_HEAD_DIM:
            raise ValueError(f"head size {self.d}: the float32 attention kernel takes any size up to "
                             f"{ops.ATTN_F32_MAX_HEAD_DIM}")
        self.qkv_bias, self.out_bias = bool(qkv_bias), bool(out_bias)
        self.window = int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.d)
        self.prefix = prefix
        n = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        # one table per distinct position encoding of the model
        pos_spec = position or PartSpec("none", {})
        shared = shared if shared is not None else {}
        key = "position:" + pos_spec.key()
        if key not in shared:
            shared[key] = POSITIONS.build(pos_spec, rt=rt)
        self.position = shared[key]
        self.w_qkv = self.b_qkv = self.b_qkv_lowp = self.w_o = self.b_o = self.p_qkv = self.p_o = None
        self._direct_loads: Optional[bool] = None     # asked of the kernel library at the first planned step

    @property
    def replayable(self) -> bool:
        # the decoding kernels cut the keys from positions in device memory; a group of more than 16 query heads
        # takes the kernel whose work items the host plans anew every step
        return self.nh // self.nkv <= DECODE_MAX_GROUP and bool(getattr(self.position, "replayable", False))

    # -- what the cache manager must hold for this mixer --------------------
    def cache_need(self) -> Optional[CacheNeed]:
        """A page holds a token's keys as [kv head][slot][D] and its values transposed, [kv head][D][slot], so that
        one read of a kv head's page serves all the query heads of its group and the kernels read four keys of one
        dim with one load; in the runtime's dtype.  The 16-bit kernels read keys 16 at a time, from one page."""
        return CacheNeed((PageTensor("k", (self.nkv, self.d), slot_axis=1), PageTensor("v", (self.nkv, self.d), slot_axis=2)),
                         window=self.window, page_multiple=16 if self.rt.lowp else 1)

    def state_need(self) -> Optional[StateNeed]:
        return None

    # -- weights -------------------------------------------------------------
    def tensors(self) -> Dict[str, TensorDecl]:
        nm, d = self.names, self.d
        t = {
            nm["q"] + ".weight": TensorDecl((self.nh * d, self.width), "matrix"),
            nm["k"] + ".weight": TensorDecl((self.nkv * d, self.width), "matrix"),
            nm["v"] + ".weight": TensorDecl((self.nkv * d, self.width), "matrix"),
            nm["o"] + ".weight": TensorDecl((self.width, self.nh * d), "matrix"),
        }
        if self.qkv_bias:
            t[nm["q"] + ".bias"] = TensorDecl((self.nh * d,), "bias")
            t[nm["k"] + ".bias"] = TensorDecl((self.nkv * d,), "bias")
            t[nm["v"] + ".bias"] = TensorDecl((self.nkv * d,), "bias")
        if self.out_bias:
            t[nm["o"] + ".bias"] = TensorDecl((self.width,), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        self.w_qkv = torch.cat([rt.place(get(nm[k] + ".weight"), "matrix") for k in "qkv"], dim=0).contiguous()
        if self.qkv_bias:
            self.b_qkv = torch.cat([rt.place(get(nm[k] + ".bias"), "bias") for k in "qkv"], dim=0).contiguous()
            self.b_qkv_lowp = self.b_qkv.to(rt.dtype)
        self.w_o = rt.place(get(nm["o"] + ".weight"), "matrix")
        if self.out_bias:
            self.b_o = rt.place(get(nm["o"] + ".bias"), "bias")
        self.p_qkv, self.p_o = rt.pack(self.w_qkv), rt.pack(self.w_o)
        self.w_qkv, self.w_o = rt.row_major(self.w_qkv, self.p_qkv), rt.row_major(self.w_o, self.p_o)

    # -- one step --------------------------------------------------------------
    def _decode_key(self):
        # what the cut of a decoding step's keys depends on: layers that agree in these share one
        return ("attention.decode_chunk", self.nkv, self._direct(), self.window)

    def _items_key(self):
        return ("attention.items", self.nh // self.nkv, self.window, self.nkv, self.d)

    def _direct(self) -> bool:
        """Whether this head size's bfloat16 kernels load keys and values straight into LDS: the host cuts their
        work differently then."""
        if self._direct_loads is None:
            self._direct_loads = ops.attention_bf16_direct(self.d)
        return self._direct_loads

    def prepare_step(self, ctx) -> Optional[Dict[tuple, np.ndarray]]:
        """The integers that this step's bfloat16 attention launches read from device memory.  A decoding step
        (one token per entry): the number of keys per work item, one integer, so that a captured step can be
        replayed with another one.  Any other step: the work items of the planned kernels.  Layers of the same
        shape share one plan."""
        if not self.rt.lowp:
            return None
        if ctx.single_token and self.nh // self.nkv <= DECODE_MAX_GROUP:
            key = self._decode_key()
            if key in ctx.extra_host:
                return None
            # (cut from the whole lengths also where a window hides most keys: the kernel numbers an entry's ranges
            # from its first key, range p holds keys p * chunk .. and p stays below p_max only if chunk covers them all)
            chunk = decode_chunk(ctx.h_kv_lens, decode_parts_max(ctx.n_positions), n_kv=self.nkv,
                                 want_blocks=DECODE_BLOCKS_DIRECT if self._direct() else DECODE_BLOCKS)
            return {key: np.array([chunk], np.int32)}
        key = self._items_key()
        if key in ctx.extra_host:
            return None
        host = plan_step(ctx.h_entry_start, ctx.h_entry_pos0, self.nh // self.nkv, self.window, self.nkv, self.d,
                         direct=self._direct())
        ctx.memo[key] = host
        return {key: host.flat()}

    def _plan(self, ctx):
        """The step's plan on the device (made once per step and shape of layer)."""
        key = self._items_key()
        plan = ctx.memo.get(("device",) + key)
        if plan is None:
            if key not in ctx.extra:
                raise RuntimeError("the attention mixer was not asked to prepare this step (prepare_step)")
            plan = device_plan(ctx.memo[key], ctx.extra[key], self.rt, self.nkv, self.d)
            ctx.memo[("device",) + key] = plan
        return plan

    def forward(self, x, ctx, cache, state=None, residual: Optional[torch.Tensor] = None, hand_on=None):
        rt, nh, nkv, d = self.rt, self.nh, self.nkv, self.d
        n = x.shape[0]
        nq = nh * d
        if cache.writes:
            qkv = linear(rt, x, self.w_qkv, self.b_qkv, "attn.qkv", bias_lowp=self.b_qkv_lowp, packed=self.p_qkv)
        else:  # keys and values of another layer: only queries are made
            bq = self.b_qkv[:nq] if self.b_qkv is not None else None
            bql = self.b_qkv_lowp[:nq] if self.b_qkv_lowp is not None else None
            qkv = linear(rt, x, self.w_qkv[:nq] if self.w_qkv is not None else None, bq, "attn.qonly", bias_lowp=bql,
                         packed=self.p_qkv.first_rows(nq) if self.p_qkv is not None else None)
        tables = self.position.rotary_tables(ctx.n_positions)
        if tables is None and hasattr(self.position, "apply") and self.position.dim != 0:
            # a position encoding that is not a plain rotation: it rewrites queries and keys with whatever it brings
            # (kernels of its own, or torch as the tests' toy does), in the projection's scratch buffer; they are then
            # stored unrotated
            qv = qkv[:, :nq].view(n, nh, d)
            kv = qkv[:, nq:nq + nkv * d].view(n, nkv, d) if cache.writes else None
            q2, k2 = self.position.apply(qv, kv, ctx.positions)
            if q2 is not qv:
                qv.copy_(q2)
            if cache.writes and k2 is not kv:
                kv.copy_(k2)
        cos, sin = tables if tables is not None else (None, None)
        plain_positions = tables is not None or getattr(self.position, "dim", 0) == 0
        chunk = ctx.extra.get(self._decode_key()) if rt.lowp and ctx.single_token else None
        p_max = decode_parts_max(ctx.n_positions)
        if (chunk is not None and cache.writes and qkv.dtype == torch.float32
                and plain_positions and (cos is None or cos.shape[1] % 8 == 0)):
            # one token per entry, straight from the projection: the attention kernel rotates and writes the pages
            out = rt.buffer("attn.out", (n, nq), rt.dtype)
            part_o = rt.buffer("attn.dec_part_o", (n * p_max * nkv * 16 * d,), torch.float32)
            part_ml = rt.buffer("attn.dec_part_ml", (n * p_max * nkv * 32,), torch.float32)
            ops.attention_bf16_decode_fused(qkv, cos, sin, cache["k"], cache["v"], cache.block_table, ctx.entry_pos0,
                                            chunk, p_max, out, part_o, part_ml, nh, nkv, d, self.window, self.scale)
            return linear(rt, out, self.w_o, self.b_o, "attn.o", packed=self.p_o, residual=residual, hand_on=hand_on)
        q = rt.buffer("attn.q", (n, nq), rt.dtype)
        ops.rope_store(qkv, cos, sin, ctx.positions, ctx.tok_entry, cache.block_table, q, cache["k"], cache["v"], nh, nkv, d,
                       write_kv=cache.writes)
        out = rt.buffer("attn.out", (n, nq), rt.dtype)
        if rt.dtype == torch.float32:
            ops.attention_f32(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, out, nh, nkv, d,
                              self.window, self.scale)
        elif chunk is not None:
            # one token per entry: the kernel cuts the keys itself from the positions on the device
            part_o = rt.buffer("attn.dec_part_o", (n * p_max * nkv * 16 * d,), torch.float32)
            part_ml = rt.buffer("attn.dec_part_ml", (n * p_max * nkv * 32,), torch.float32)
            ops.attention_bf16_decode(q, cache["k"], cache["v"], cache.block_table, ctx.entry_pos0, chunk, p_max, out,
                                      part_o, part_ml, nh, nkv, d, self.window, self.scale)
        else:
            plan = self._plan(ctx)
            if plan.n_items:        # decoded tokens and short portions: 16-row items, keys split where that helps
                ops.attention_bf16(q, cache["k"], cache["v"], cache.block_table, plan.items, plan.n_items, plan.citems,
                                   plan.n_citems, out, plan.part_o, plan.part_ml, nh, nkv, d, self.window, self.scale,
                                   max_part=plan.n_parts, rt=plan.rt)
            if plan.n_tile_items:   # long portions: key/value blocks through LDS, shared by four waves
                ops.attention_bf16_tiles(q, cache["k"], cache["v"], cache.block_table, plan.tile_items, plan.n_tile_items,
                                         out, nh, nkv, d, self.window, self.scale, rt=plan.tile_rt,
                                         citems=plan.tile_citems, n_citems=plan.n_tile_citems,
                                         part_o=plan.tile_part_o, part_ml=plan.tile_part_ml, n_parts=plan.n_tile_parts)
        return linear(rt, out, self.w_o, self.b_o, "attn.o", packed=self.p_o, residual=residual, hand_on=hand_on)
