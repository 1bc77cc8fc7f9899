"""Sampling options of a request: the names, defaults and meanings of the
reference's front end (sglfront/sglfront/core.py:6-16), plus a seed."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    temperature: float = 0.0   # <= 0: greedy
    top_k: int = -1            # -1: no cut; 1: greedy
    top_p: float = 1.0         # 1.0: no cut
    ignore_eos: bool = False
    max_tokens: int = 1024
    seed: Optional[int] = None  # None: derived from the engine's seed and the request's id

    def __post_init__(self):
        if self.max_tokens < 1:
            raise ValueError(f"max_tokens must be at least 1, got {self.max_tokens}")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if self.top_k == 0 or self.top_k < -1:
            raise ValueError(f"top_k must be -1 (off) or positive, got {self.top_k}")

    @property
    def is_greedy(self) -> bool:
        return (self.temperature <= 0.0 or self.top_k == 1) and self.top_p == 1.0
