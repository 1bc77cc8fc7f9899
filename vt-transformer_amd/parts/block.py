"""Arrangement of a layer's parts around the residual stream.

"prenorm" is the reference's layer (v1/models/qwen2-7b/inference_fp16.dag:287-345):
norm -> mixer -> add -> norm -> feed-forward -> add.  The residual stream h is
fp32.  A layer hands its last output on unadded (`delta`), so the next norm
adds it in the same kernel that normalises.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import BLOCKS, Part, Runtime


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    norm_roles = ("input", "post_mixer")

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward):
        self.rt = rt
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]
        self.mixer = mixer
        self.feed_forward = feed_forward

    def parts(self):
        return [self.norm_in, self.mixer, self.norm_post, self.feed_forward]

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache, state) -> Tuple[torch.Tensor, torch.Tensor]:
        a = self.norm_in.forward(h, delta)
        y = self.mixer.forward(a, ctx, cache, state)
        b = self.norm_post.forward(h, y)
        z = self.feed_forward.forward(b, ctx)
        return h, z
