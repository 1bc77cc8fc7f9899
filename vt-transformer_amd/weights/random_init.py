"""Random weights from a configuration and a seed.

The reference has no such mode (its nearest thing is the fixed generator
mt19937(1979) of v1/tensortype/context.cpp:45).  Matrices and biases are
N(0, 0.02), norm gains 1 + N(0, 0.02); each tensor is drawn from a generator
seeded by (seed, tensor name), so the values of a tensor do not depend on
which other tensors exist or in which order they are made.
"""
from __future__ import annotations

import hashlib
import os
from typing import Dict, Iterator, Tuple

import torch

from ..config.base import ModelConfig
from ..parts.base import Runtime, TensorDecl
from .safetensors_io import write_safetensors

STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, decl: TensorDecl, seed: int, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    g = torch.Generator(device=device)
    g.manual_seed(_tensor_seed(seed, name))
    if decl.role == "table":
        return torch.zeros(decl.shape, dtype=torch.int32, device=device)
    t = torch.randn(decl.shape, generator=g, dtype=torch.float32, device=device) * STD
    if decl.role == "gain":
        t += 1.0
    return t.to(dtype)


def random_tensors(expected: Dict[str, TensorDecl], seed: int, device: torch.device,
                   dtype: torch.dtype) -> Iterator[Tuple[str, torch.Tensor]]:
    for name, decl in expected.items():
        if decl.optional:
            continue
        yield name, random_tensor(name, decl, seed, device, dtype)


def declared_tensors(config: ModelConfig) -> Dict[str, TensorDecl]:
    """The tensors a model of this configuration loads (no device is touched)."""
    from ..models.model import DecoderModel
    model = DecoderModel(config.to_spec(), Runtime(torch.device("cpu"), torch.float32))
    return model.tensors()


def write_random_model(config: ModelConfig, folder: str, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """Write config.json and model.safetensors with random weights; returns the folder."""
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    expected = declared_tensors(config)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(expected, seed, torch.device("cpu"), dtype),
                      metadata={"format": "pt", "seed": seed})
    return folder
