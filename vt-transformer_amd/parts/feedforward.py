"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases.

The reference's order (v1/models/qwen2-7b/inference_fp16.dag:333-337): up
projection (mlp.w2), gate projection (mlp.w1), silu(gate) * up
(v1/tensortype/hip_kernels/silu_product.cpp:8-16), down projection
(mlp.o_proj); w1 = gate_proj, w2 = up_proj, o_proj = down_proj
(v1/models/qwen2-7b/dump_from_huggingface.py:89-99).  Gate and up are one
matrix here (gate rows, then up rows); with few tokens the gating is applied
to the fp32 accumulators inside the product's kernel.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, Part, Runtime, TensorDecl
from .base import NormedInput
from .linear import GATED_MAX_ROWS, UNPACK_MIN_ROWS, can_add_residual, can_fuse, linear, takes_prepared_norm


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, width: int, prefix: str, intermediate_size: int, activation: str = "silu",
                 names: Optional[Dict[str, str]] = None):
        if activation != "silu":
            raise ValueError(f"activation '{activation}' is not supported (only 'silu')")
        self.rt = rt
        self.width = int(width)
        self.inter = int(intermediate_size)
        n = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.w_gu = self.w_down = self.p_gu = self.p_down = None

    def tensors(self) -> Dict[str, TensorDecl]:
        nm = self.names
        return {
            nm["gate"] + ".weight": TensorDecl((self.inter, self.width), "matrix"),
            nm["up"] + ".weight": TensorDecl((self.inter, self.width), "matrix"),
            nm["down"] + ".weight": TensorDecl((self.width, self.inter), "matrix"),
        }

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        self.w_gu = torch.cat([rt.place(get(nm["gate"] + ".weight"), "matrix"),
                               rt.place(get(nm["up"] + ".weight"), "matrix")], dim=0).contiguous()
        self.w_down = rt.place(get(nm["down"] + ".weight"), "matrix")
        self.p_gu, self.p_down = rt.pack(self.w_gu, halves=2), rt.pack(self.w_down)
        self.w_gu, self.w_down = rt.row_major(self.w_gu, self.p_gu), rt.row_major(self.w_down, self.p_down)

    takes_normed_input = True     # the gate/up product applies the norm in front of it when the rows are few
    hands_norm_on = True          # ... and the down product prepares the norm behind it

    def adds_residual(self, rows: int) -> bool:
        """Whether the down product adds to the residual stream itself at this many rows."""
        return can_add_residual(self.rt, rows, self.width, self.inter)

    def forward(self, x, ctx=None, residual: Optional[torch.Tensor] = None, hand_on=None):
        rt = self.rt
        n = x.shape[0]
        act = rt.buffer("mlp.act", (n, self.inter), rt.dtype)
        normed = isinstance(x, NormedInput)
        if normed:
            ok = (takes_prepared_norm(rt, n, self.width) and self.p_gu is not None) if x.prepared else \
                (can_fuse(rt, n) and self.width % 8 == 0)
            if not ok:
                x, normed = x.materialize(), False
        if rt.lowp and (n <= GATED_MAX_ROWS or (self.w_gu is None and (rt.keep_row_major or n < UNPACK_MIN_ROWS))):
            w = self.p_gu if self.p_gu is not None else self.w_gu
            if normed and x.prepared:
                ops.gated_linear_bf16_link(x.xn, w, act, x.ssq, x.eps)
            elif normed:
                ops.gated_linear_bf16(x.h, w, act, norm_gain=x.gain, norm_eps=x.eps)
            else:
                ops.gated_linear_bf16(x, w, act)
        else:
            gu = linear(rt, x, self.w_gu, None, "mlp.gu", packed=self.p_gu if self.w_gu is None else None)
            ops.silu_mul(gu, act)
        return linear(rt, act, self.w_down, None, "mlp.down", packed=self.p_down, residual=residual, hand_on=hand_on)
