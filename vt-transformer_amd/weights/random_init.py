"""Random weights from a configuration and a seed.

The reference has no such mode (its nearest thing is the fixed generator
mt19937(1979) of v1/tensortype/context.cpp:45).  Matrices and biases are
close to N(0, 0.02), norm gains 1 + N(0, 0.02).  Every element is a function
of (seed, tensor name, index of the element) alone: a counter-based generator
(three words of a SplitMix64 stream, cut into twelve 16-bit integers whose
sum stands in for a normal deviate: exact integer arithmetic, then one
multiplication and one addition in float32).  The values therefore do not
depend on which other tensors exist, in which order or in which pieces they
are made, or where: `counter_normal` on the host and the kernel
`vt_random_normal` on the device give the same bits, so a model drawn on the
device (`random_model`, which never exists on the host) is the model that
`write_random_model` stores for the same seed.
"""
from __future__ import annotations

import hashlib
import os
from typing import Dict, Iterator, Tuple

import numpy as np
import torch

from ..config.base import ModelConfig
from ..parts.base import Runtime, TensorDecl
from .safetensors_io import write_safetensors

STD = 0.02

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_SUM_MEAN = 393210                                   # twelve 16-bit integers: 12 * 65535 / 2
_SUM_STD = float(np.sqrt(np.float64(2 ** 32 - 1)))   # sqrt(12 * (65536^2 - 1) / 12)


def tensor_key(seed: int, name: str) -> int:
    """64 bits that stand for (seed, tensor name)."""
    return int.from_bytes(hashlib.sha256(f"{seed}:{name}".encode()).digest()[:8], "little")


def normal_scale(std: float) -> float:
    """The float32 factor that turns the centred sum of integers into a deviate of this standard deviation."""
    return float(np.float32(std / _SUM_STD))


def counter_normal(key: int, first: int, n: int, std: float, mean: float) -> np.ndarray:
    """Elements first .. first + n - 1 of the stream of `key`, float32: the host's twin of vt_random_normal."""
    with np.errstate(over="ignore"):
        e = np.arange(first, first + n, dtype=np.uint64)
        total = np.zeros(n, dtype=np.int64)
        for j in (1, 2, 3):
            z = np.uint64(key) + (np.uint64(3) * e + np.uint64(j)) * _GAMMA
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            z = z ^ (z >> np.uint64(31))
            for shift in (0, 16, 32, 48):
                total += ((z >> np.uint64(shift)) & np.uint64(0xFFFF)).astype(np.int64)
    centred = (total - _SUM_MEAN).astype(np.float32)
    return centred * np.float32(normal_scale(std)) + np.float32(mean)


_HOST_PIECE = 1 << 22      # elements made at a time on the host


def random_tensor(name: str, decl: TensorDecl, seed: int, device: torch.device, dtype: torch.dtype) -> torch.Tensor:
    """The tensor `name` of the model with this seed, on `device` (the GPU's kernel or the host's twin: same bits)."""
    if decl.role == "table":
        return torch.zeros(decl.shape, dtype=torch.int32, device=device)
    key = tensor_key(seed, name)
    mean = 1.0 if decl.role == "gain" else 0.0
    n = 1
    for d in decl.shape:
        n *= int(d)
    if torch.device(device).type == "cuda":
        from ..kernels import ops
        out = torch.empty(decl.shape, dtype=dtype, device=device)
        return ops.random_normal(out, key, normal_scale(STD), mean)
    out = torch.empty(n, dtype=dtype)
    for first in range(0, n, _HOST_PIECE):
        m = min(_HOST_PIECE, n - first)
        out[first:first + m] = torch.from_numpy(counter_normal(key, first, m, STD, mean)).to(dtype)
    return out.reshape(decl.shape)


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
