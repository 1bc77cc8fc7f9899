"""Rotary position encoding: the table of angles.

The reference builds it on the host (v1/tensortype/common.cpp:6-24):
inv_freq[i] = 1 / base^(2i/D) for i < D/2, the angle of position l is
l * inv_freq[i], and the table holds its cosine and sine as floats.  Dims i
and i + D/2 share an angle and form a rotated pair
(v1/tensortype/hip_kernels/rotary_embed.cpp:20-26); the rotation itself is
fused into the kernel that writes keys and values into their pages.

The reference rounds inv_freq and the angle to float before taking cosine
and sine, which costs about position * 1e-7 radians; here everything up to
the final cosine and sine is computed in double and rounded to float once.
The reference's table has 10000 rows (v1/models/qwen2-7b/inference_fp16.dag:38);
here it has as many as the longest sequence the engine is set up for.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from .base import POSITIONS, Part, Runtime


def rotary_table(n_positions: int, dims: int, theta: float) -> Tuple[np.ndarray, np.ndarray]:
    """(cos, sin), float32 [n_positions, dims/2]."""
    i = np.arange(0, dims, 2, dtype=np.float64)
    inv = 1.0 / np.power(np.float64(theta), i / dims)
    ang = np.arange(n_positions, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


@POSITIONS.register("rotary")
class RotaryEncoding(Part):
    replayable = True

    def __init__(self, *, rt: Runtime, theta: float, dim: int):
        if dim % 2:
            raise ValueError(f"rotary dims {dim} must be even")
        self.rt = rt
        self.theta = float(theta)
        self.dim = int(dim)
        self._tables: Optional[Tuple[torch.Tensor, torch.Tensor]] = None

    def rotary_tables(self, n_positions: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """fp32 cos and sin [>= n_positions, dim/2] on the device, for the fused kernel."""
        if self._tables is None or self._tables[0].shape[0] < n_positions:
            cos, sin = rotary_table(n_positions, self.dim, self.theta)
            self._tables = (torch.from_numpy(cos).to(self.rt.device), torch.from_numpy(sin).to(self.rt.device))
        return self._tables


@POSITIONS.register("none")
class NoPositionEncoding(Part):
    replayable = True

    """Queries and keys as they are."""

    def __init__(self, *, rt: Runtime):
        self.rt = rt
        self.dim = 0

    def rotary_tables(self, n_positions: int):
        return None

    def apply(self, q, k, positions):
        return q, k
