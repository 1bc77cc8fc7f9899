from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, CacheNeed, PageTensor, Part,
                   Registry, Runtime, StateNeed, TensorDecl)
from . import norm, rotary, attention, feedforward, block, embedding  # noqa: F401  (register the built-in parts)

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "CacheNeed", "PageTensor",
           "Part", "Registry", "Runtime", "StateNeed", "TensorDecl"]
