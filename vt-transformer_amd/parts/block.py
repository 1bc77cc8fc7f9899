"""Arrangement of a layer's parts around the residual stream.

"prenorm" is the reference's layer (v1/models/qwen2-7b/inference_fp16.dag:287-345):
norm -> mixer -> add -> norm -> feed-forward -> add.  The residual stream h is
fp32.  A layer hands its last output on unadded (`delta`), so the next norm
adds it in the same kernel that normalises.

With few rows in bfloat16 (decoding) the norms and additions are not kernels of
their own: a mixer or feed-forward that says so takes the residual stream with
the norm still to be applied (`NormedInput`: its first matrix product applies
it) and adds its result to the stream itself (`residual=`: its last matrix
product does; `adds_residual(rows)` says for how many rows it can, which reaches
up to 64 for matrices that fill the GPU without splitting k over blocks).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import BLOCKS, NormedInput, Part, Runtime
from .linear import can_fuse
from .norm import RMSNorm


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    norm_roles = ("input", "post_mixer")
    replayable = True

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward):
        self.rt = rt
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]
        self.mixer = mixer
        self.feed_forward = feed_forward

    def parts(self):
        return [self.norm_in, self.mixer, self.norm_post, self.feed_forward]

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache, state) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        fuse = can_fuse(self.rt, h.shape[0]) and h.shape[1] % 8 == 0
        y = self._run(self.mixer, self.norm_in, h, delta, fuse, ctx, cache, state)
        z = self._run(self.feed_forward, self.norm_post, h, y, fuse, ctx)
        return h, z

    def _run(self, part, norm, h, delta, fuse, *args):
        """norm (of h + delta), then the part; returns what is still to be added to h (None: the part added it)."""
        if fuse and delta is None and isinstance(norm, RMSNorm) and getattr(part, "takes_normed_input", False):
            x = NormedInput(h, norm)
        else:
            x = norm.forward(h, delta)
        adds = getattr(part, "adds_residual", None)
        if adds is not None and adds(h.shape[0]):
            part.forward(x, *args, residual=h)
            return None
        return part.forward(x, *args)
