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

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
        raise ValueError(f"dtype {name} is not supported (bfloat16 and float32 are)")
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype '{name}' is not supported (bfloat16 and float32 are)") from None


def build_model(config: ModelConfig, dtype, device: Optional[torch.device] = None,
                keep_row_major: bool = True) -> DecoderModel:
    device = device or require_gpu()
    return DecoderModel(config.to_spec(), Runtime(device, parse_dtype(dtype), keep_row_major))


def load_model(folder: str, dtype, device: Optional[torch.device] = None, keep_row_major: bool = True) -> DecoderModel:
    """config.json chooses the architecture; model.safetensors (or its shards) gives the tensors."""
    model = build_model(load_config(folder), dtype, device, keep_row_major)
    load_model_weights(model, folder)
    return model


def random_model(config: ModelConfig, seed: int, dtype, device: Optional[torch.device] = None,
                 keep_row_major: bool = True) -> DecoderModel:
    """The same tensors that `write_random_model` would store for this seed's generator on this device,
    drawn on the device one at a time (a 145 GB model never exists on the host)."""
    model = build_model(config, dtype, device, keep_row_major)
    expected = model.tensors()
    rt = model.rt

    def get(name: str) -> torch.Tensor:
        return random_tensor(name, expected[name], seed, rt.device, torch.bfloat16)
    model.load(get)
    return model


def make_runner(model: DecoderModel, *, pool_tokens: int, page_size: int = 16, max_requests: int = 64,
                max_seq_len: Optional[int] = None) -> ModelRunner:
    if model.rt.dtype == torch.bfloat16 and page_size % 16:
        raise ValueError(f"page size {page_size}: the bfloat16 attention kernel reads keys 16 at a time, "
                         f"the page size must be a multiple of 16")
    if max_seq_len is None:
        max_seq_len = min(model.spec.max_positions, max(pool_tokens, page_size))
    return ModelRunner(model, model.rt, page_size, pool_tokens, max_requests, max_seq_len)
