"""A decoder put together from a `ModelSpec`: embedding, layers, the order in
which they run, final norm and head.  It is the same class for every
architecture; what differs is the spec.

The reference's counterpart is the outer program gpu_main
(v1/models/qwen2-7b/inference_fp16.dag:368-396): embed, 28 x layer_forward,
final norm over the rows, logits where the mask asks for them.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..config.base import LayerSpec, ModelSpec, PartSpec
from ..parts.base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, NormedInput, Part, Registry,
                          Runtime, TensorDecl)


def build_part(registry: Registry, spec: PartSpec, prefix: str, **context):
    params = dict(spec.params)
    local = params.pop("prefix", "")
    return registry.build(PartSpec(spec.kind, params), prefix=prefix + local, **context)


class DecoderModel:
    def __init__(self, spec: ModelSpec, rt: Runtime):
        spec.validate()
        self.spec = spec
        self.rt = rt
        width = spec.hidden_size
        shared: dict = {}  # parts that several layers hold one instance of (position tables)
        self.embedding = EMBEDDINGS.build(spec.embedding, rt=rt, width=width, vocab_size=spec.vocab_size)
        self.layers = [self._build_layer(ls, shared) for ls in spec.layers]
        self.final_norm = build_part(NORMS, spec.final_norm, "", rt=rt, width=width)
        self.head = HEADS.build(spec.head, rt=rt, width=width, vocab_size=spec.vocab_size)
        self.schedule = list(spec.schedule)

    def _build_layer(self, ls: LayerSpec, shared: dict):
        rt, width = self.rt, self.spec.hidden_size
        norms = {role: build_part(NORMS, ns, ls.prefix, rt=rt, width=width) for role, ns in ls.norms.items()}
        mixer = build_part(MIXERS, ls.mixer, ls.prefix, rt=rt, width=width, shared=shared)
        ffn = build_part(FEED_FORWARDS, ls.feed_forward, ls.prefix, rt=rt, width=width)
        return BLOCKS.build(ls.block, rt=rt, norms=norms, mixer=mixer, feed_forward=ffn)

    # ------------------------------------------------------------------
    def parts(self) -> List[Part]:
        out: List[Part] = [self.embedding]
        for layer in self.layers:
            out.extend(layer.parts())
        out.extend([self.final_norm, self.head])
        return out

    def tensors(self) -> Dict[str, TensorDecl]:
        out: Dict[str, TensorDecl] = {}
        for p in self.parts():
            for name, decl in p.tensors().items():
                if name in out and out[name].shape != decl.shape:
                    raise ValueError(f"tensor '{name}' is declared twice with shapes {out[name].shape} and {decl.shape}")
                if name not in out or not decl.optional:
                    out[name] = decl
        return out

    def load(self, get: Callable[[str], torch.Tensor]) -> None:
        self.embedding.load(get, self.rt)
        for layer in self.layers:
            for p in layer.parts():
                p.load(get, self.rt)
        self.final_norm.load(get, self.rt)
        # a head's loader takes `shared`: tensors by name that other parts have already placed on the device (the
        # embedding's table, which a tied head multiplies by)
        shared = {}
        if getattr(self.embedding, "table", None) is not None:
            shared[self.embedding.name] = self.embedding.table
        self.head.load(get, self.rt, shared=shared)

    # ------------------------------------------------------------------
    def forward(self, ctx, caches, states) -> Optional[torch.Tensor]:
        """Run the tokens of one step.  caches[i] / states[i] belong to schedule entry i.
        Returns fp32 logits [rows wanted, vocab], or None if no row is wanted."""
        h = self.embedding.forward(ctx.token_ids)
        delta = None
        last = len(self.schedule) - 1
        for i, entry in enumerate(self.schedule):
            block = self.layers[entry.layer]
            if getattr(block, "takes_next_norm", False):
                # the norm that the layer behind starts with, which this layer's last product may prepare
                nxt = getattr(self.layers[self.schedule[i + 1].layer], "first_norm", None) if i < last else None
                h, delta = block.forward(h, delta, ctx, caches[i], states[i], next_norm=nxt)
            else:
                if isinstance(delta, NormedInput):
                    delta = None            # (its addition is done; this block applies its own norm)
                h, delta = block.forward(h, delta, ctx, caches[i], states[i])
        if ctx.n_logit_rows == 0:
            return None
        if isinstance(delta, NormedInput):
            delta = None
        x = self.final_norm.forward(h, delta, rows=ctx.logit_rows)
        return self.head.forward(x)
