"""Choosing next tokens from logits, one row per request.

The choice itself is a HIP kernel (greedy, or temperature with top_k / top_p
and the inverse CDF).  The uniform number of a draw comes from the host, as
in the reference (one `randx` per call, v1/tensortype/hip_tensor.cpp:1033-1034),
but from a counter-based generator keyed by (request seed, index of the
token in the request's output): a request draws the same numbers whatever
else is in the batch and however often it was preempted.
"""
from __future__ import annotations

import hashlib
from typing import List, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from ..parts.base import HostStaging, Runtime
from .params import SamplingParams

_M64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _M64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform(seed: int, counter: int) -> float:
    """A number in [0, 1) that depends only on (seed, counter); 24 bits, exact in float32."""
    z = _splitmix64(_splitmix64(seed & _M64) ^ ((counter * 0xD1342543DE82EF95) & _M64))
    return (z >> 40) / float(1 << 24)


def request_seed(engine_seed: int, request_key) -> int:
    """The same for the same (engine seed, request id) in every process (Python's own hash of a string is not)."""
    key = int.from_bytes(hashlib.sha256(str(request_key).encode()).digest()[:8], "little")
    return _splitmix64((engine_seed & _M64) ^ _splitmix64(key))


class Pending:
    """Tokens that have been chosen on the device and are on their way to the host."""

    def __init__(self, tokens_dev: torch.Tensor, host: torch.Tensor, event, rows: int):
        self.tokens_dev, self.host, self.event, self.rows = tokens_dev, host, event, rows


class Sampler:
    def __init__(self, rt: Runtime):
        self.rt = rt
        self._staging = HostStaging(torch.float32)
        self._turn = 0
        self._host: dict = {}

    def sample(self, logits: torch.Tensor, rows: Sequence[Tuple[SamplingParams, int, int]]) -> List[int]:
        """logits [R, V] fp32 on the device; rows[i] = (params, seed, counter) of row i."""
        return self.collect(self.launch(logits, rows))

    def collect(self, pending: Pending) -> List[int]:
        pending.event.synchronize()
        return pending.host[:pending.rows].tolist()

    def launch(self, logits: torch.Tensor, rows: Sequence[Tuple[SamplingParams, int, int]]) -> Pending:
        """Choose the tokens and start their copy to the host without waiting for either: `collect` waits.  The
        tokens also stay on the device (`tokens_dev`) for a next step that starts before the host has read them.
        Two sets of buffers take turns, so one launch may be outstanding while the next is made."""
        r, v = logits.shape
        if r != len(rows):
            raise ValueError(f"{r} rows of logits for {len(rows)} requests")
        host = np.zeros((4, r), dtype=np.float32)
        for i, (p, seed, counter) in enumerate(rows):
            greedy = p.temperature <= 0.0 or p.top_k == 1
            host[0, i] = 0.0 if greedy else p.temperature
            host[1, i] = p.top_p
            host[2, i] = uniform(seed, counter)
            host[3, i] = np.int32(p.top_k).view(np.float32)
        dev = self.rt.buffer("sample.params", (4, r), torch.float32)
        self._staging.upload(host, dev)
        self._turn ^= 1
        out = self.rt.buffer(f"sample.out{self._turn}", (r,), torch.int32)
        if any(host[0, i] > 0 for i in range(r)):
            work = self.rt.buffer("sample.work", (r * v,), torch.float32)   # probabilities of the stochastic rows
        else:
            work = logits.view(-1)   # greedy rows never touch the workspace
        partials = self.rt.buffer("sample.partials", (ops.sample_partials_size(r),), torch.float32)
        ops.sample(logits, dev[0], dev[3].view(torch.int32), dev[1], dev[2], work, out, partials)
        host = self._host.get(self._turn)
        if host is None or host.numel() < r:
            host = torch.empty(max(r, 64), dtype=torch.int32, pin_memory=True)
            self._host[self._turn] = host
        host[:r].copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return Pending(out, host, event, r)
