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
up to 64 for matrices that fill the GPU without splitting k over blocks).  A part
that `hands_norm_on` is also told which norm comes behind it (`hand_on=`) and
may return that norm prepared (a NormedInput with `xn` and `ssq`), which the
part behind the norm then takes as its input.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .base import BLOCKS, NormedInput, Part, Runtime
from .linear import can_fuse


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    norm_roles = ("input", "post_mixer")
    replayable = True
    takes_next_norm = True      # forward(..., next_norm=): the norm that the layer behind this one starts with

    def __init__(self, *, rt: Runtime, norms, mixer, feed_forward):
        self.rt = rt
        self.norm_in = norms["input"]
        self.norm_post = norms["post_mixer"]
        self.mixer = mixer
        self.feed_forward = feed_forward

    def parts(self):
        return [self.norm_in, self.mixer, self.norm_post, self.feed_forward]

    @property
    def first_norm(self):
        """The norm that this layer applies to the stream it is given (what the layer in front may prepare)."""
        return self.norm_in

    def forward(self, h: torch.Tensor, delta, ctx, cache, state, next_norm=None) -> Tuple[torch.Tensor, object]:
        """delta: what is still to be added to h (a tensor), None, or this layer's first norm as the layer in front
        has prepared it (a NormedInput; its addition is done).  Returns (h, delta) in the same terms."""
        fuse = can_fuse(self.rt, h.shape[0]) and h.shape[1] % 8 == 0
        y = self._run(self.mixer, self.norm_in, h, delta, fuse, self.norm_post, ctx, cache, state)
        z = self._run(self.feed_forward, self.norm_post, h, y, fuse, next_norm, ctx)
        return h, z

    def _run(self, part, norm, h, delta, fuse, norm_behind, *args):
        """norm (of h + delta), then the part; returns what is still to be added to h (None: the part added it; a
        NormedInput: it added it and prepared `norm_behind`)."""
        takes = getattr(part, "takes_normed_input", False)
        if isinstance(delta, NormedInput):
            x = delta if (delta.norm is norm and takes) else norm.forward(h, None)
        elif fuse and delta is None and getattr(norm, "rms_fusable", False) and takes:
            x = NormedInput(h, norm)
        else:
            x = norm.forward(h, delta)
        adds = getattr(part, "adds_residual", None)
        if adds is not None and adds(h.shape[0]):
            if norm_behind is not None and getattr(part, "hands_norm_on", False):
                r = part.forward(x, *args, residual=h, hand_on=norm_behind)
                return r if isinstance(r, NormedInput) else None
            part.forward(x, *args, residual=h)
            return None
        return part.forward(x, *args)
