"""RMSNorm, fused with the residual addition that precedes it.

out = (w * x) * 1/sqrt(mean(x^2) + eps), all in fp32, one rounding to the
output dtype (v1/tensortype/hip_kernels/rmsnorm.cpp:7-44: the sum of squares
divided by the width, eps inside the root, product evaluated (w*x)*r).
x = h + delta is the reference's fp32 residual addition
(v1/tensortype/hip_kernels/pointwise.cpp:51-57).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import NORMS, Part, Runtime, TensorDecl


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    replayable = True
    # out = (gain * x) / sqrt(mean(x^2) + eps) with `gain` and `eps` as attributes: a matrix product can apply it on
    # the way (NormedInput); any norm of that form may say so
    rms_fusable = True

    def __init__(self, *, rt: Runtime, width: int, prefix: str, eps: float, name: str = "weight", scratch: str = "norm"):
        self.rt = rt
        self.width = int(width)
        self.eps = float(eps)
        self.name = prefix + name
        self.scratch = scratch
        self.gain: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorDecl]:
        return {self.name: TensorDecl((self.width,), "gain")}

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        self.gain = rt.place(get(self.name), "gain")

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else h.shape[0]
        out = self.rt.buffer(self.scratch + (".rows" if rows is not None else ""), (n, self.width), self.rt.dtype)
        return ops.rmsnorm(h, delta, self.gain, out, self.eps, rows=rows)
