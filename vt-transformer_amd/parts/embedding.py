"""Token embedding and output head.

Embedding: row copy, xinput[t] = wte[ids[t]] (v1/tensortype/host_tensor.cpp:169-201,
device variant v1/tensortype/hip_kernels/embed.cpp:7-37); the rows become the
fp32 residual stream.  Head: logits = lm_head . x only for the rows that are
asked for (the reference marks them with mask value 2,
v1/tensortype/hip_tensor.cpp:923-991) and kept in fp32 here.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Part, Runtime, TensorDecl
from .linear import SKINNY_MAX_ROWS


@EMBEDDINGS.register("embedding")
class TokenEmbedding(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, width: int, vocab_size: int, name: str):
        self.rt, self.width, self.vocab, self.name = rt, int(width), int(vocab_size), name
        self.table: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name: TensorDecl((self.vocab, self.width), "matrix")}

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        self.table = rt.place(get(self.name), "matrix")

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        h = self.rt.buffer("h", (ids.numel(), self.width), torch.float32)
        return ops.embed(self.table, ids, h)


@HEADS.register("linear_head")
class LinearHead(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, width: int, vocab_size: int, name: str, tied_to: Optional[str] = None):
        self.rt, self.width, self.vocab, self.name, self.tied_to = rt, int(width), int(vocab_size), name, tied_to
        self.weight: Optional[torch.Tensor] = None
        self.packed = None

    def tensors(self) -> Dict[str, TensorDecl]:
        if self.tied_to:
            # a tied head has no tensor of its own; a stored copy is tolerated and not used
            return {self.name: TensorDecl((self.vocab, self.width), "matrix", optional=True)}
        return {self.name: TensorDecl((self.vocab, self.width), "matrix")}

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime, shared: Optional[Dict[str, torch.Tensor]] = None) -> None:
        if self.tied_to:
            if shared is None or self.tied_to not in shared:
                raise ValueError(f"head is tied to '{self.tied_to}', which no part has loaded")
            self.weight = shared[self.tied_to]
        else:
            self.weight = rt.place(get(self.name), "matrix")
        self.packed = rt.pack(self.weight)
        if self.packed is not None and not self.tied_to:
            self.weight = None      # bfloat16 logits always come from the packed matrix

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [R, H] (normed rows) -> fp32 logits [R, V]."""
        r = x.shape[0]
        out = self.rt.buffer("logits", (r, self.vocab), torch.float32)
        if self.rt.dtype == torch.float32:
            return ops.linear_f32(x, self.weight, None, out)
        for r0 in range(0, r, SKINNY_MAX_ROWS):
            r1 = min(r, r0 + SKINNY_MAX_ROWS)
            need = ops.linear_bf16_workspace(r1 - r0, self.vocab, self.width) if r1 - r0 > 16 else 0
            work = self.rt.buffer("linear.partials", (need,), torch.float32) if need else None
            ops.linear_bf16(x[r0:r1], self.packed, None, out[r0:r1], work)
        return out
