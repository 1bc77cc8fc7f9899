"""From a model folder (or a configuration and a seed) to a ModelRunner on the GPU."""
from __future__ import annotations

from typing import Optional

import torch

from ..config import ModelConfig, load_config
from ..kernels.ops import require_gpu
from ..models.model import DecoderModel
from ..parts.base import Runtime
from ..weights.loader import check_tensors, load_model_weights
from ..weights.random_init import random_tensor
from .step import ModelRunner

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float16": torch.float16, "fp16": torch.float16,
           "f16": torch.float16, "half": torch.float16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float16, torch.float32):
            return name
        raise ValueError(f"dtype {name} is not supported (bfloat16, float16 and float32 are)")
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype '{name}' is not supported (bfloat16, float16 and float32 are)") from None


def build_model(config: ModelConfig, dtype, device: Optional[torch.device] = None,
                keep_row_major: bool = True) -> DecoderModel:
    device = device or require_gpu()
    return DecoderModel(config.to_spec(), Runtime(device, parse_dtype(dtype), keep_row_major))


def load_model(folder: str, dtype, device: Optional[torch.device] = None, keep_row_major: bool = True,
               page_size: Optional[int] = None) -> DecoderModel:
    """config.json chooses the architecture; model.safetensors (or its shards) gives the tensors.  With `page_size`
    the model's parts are asked whether they take it before any tensor is read."""
    model = build_model(load_config(folder), dtype, device, keep_row_major)
    if page_size is not None:
        check_page_size(model, page_size)
    load_model_weights(model, folder)
    return model


def random_model(config: ModelConfig, seed: int, dtype, device: Optional[torch.device] = None,
                 keep_row_major: bool = True, page_size: Optional[int] = None) -> DecoderModel:
    """The tensors that `write_random_model` stores for this seed (the same bits: one counter-based generator, on
    the host there and on the device here), drawn on the device one at a time: a 145 GB model never exists on the
    host."""
    model = build_model(config, dtype, device, keep_row_major)
    if page_size is not None:
        check_page_size(model, page_size)
    expected = model.tensors()
    rt = model.rt

    def get(name: str) -> torch.Tensor:
        return random_tensor(name, expected[name], seed, rt.device, torch.bfloat16)
    model.load(get)
    return model


def check_page_size(model: DecoderModel, page_size: int) -> None:
    """What the model's mixers refuse in a page size (CacheNeed.page_multiple), said before anything is loaded or run."""
    if page_size <= 0:
        raise ValueError(f"page size {page_size} must be positive")
    for layer in model.layers:
        need = layer.mixer.cache_need() if hasattr(layer.mixer, "cache_need") else None
        if need is not None and page_size % max(1, need.page_multiple):
            raise ValueError(f"page size {page_size}: the {str(model.rt.dtype).replace('torch.', '')} kernels of "
                             f"{type(layer.mixer).__name__} read keys {need.page_multiple} at a time, the page size "
                             f"must be a multiple of {need.page_multiple}")


def make_runner(model: DecoderModel, *, pool_tokens: Optional[int] = None, page_size: int = 16, max_requests: int = 64,
                max_seq_len: Optional[int] = None, kv_bytes: Optional[int] = None,
                max_portion: Optional[int] = None) -> ModelRunner:
    """The cache's size is `pool_tokens` (tokens that each group of layers holds) or `kv_bytes` (bytes for all pages
    together, shared by the groups by their needs: a group with a window gets pages for its window and `max_portion`
    tokens, the most of one request that a step will bring, per request; the rest goes to the groups that keep
    every key)."""
    check_page_size(model, page_size)
    if max_seq_len is None:
        if pool_tokens is None:
            max_seq_len = model.spec.max_positions
        else:
            max_seq_len = min(model.spec.max_positions, max(pool_tokens, page_size))
    return ModelRunner(model, model.rt, page_size, pool_tokens, max_requests, max_seq_len, kv_bytes=kv_bytes,
                       max_portion=max_portion)
