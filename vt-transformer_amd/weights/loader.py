"""Loading a model's tensors by name, with one error for everything that does
not fit.

The reference loads one raw file per tensor and asserts its size
(v1/tensortype/hip_tensor.cpp:61-71), under names that its dump script derives
from the checkpoint's (v1/models/qwen2-7b/dump_from_huggingface.py:47-99);
here the checkpoint's own names are the keys, as in the newer
vt-transformer/models/qwen3-0.6b/init.vt:39-62.
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..parts.base import TensorDecl
from .safetensors_io import WeightStore


class WeightError(ValueError):
    """Tensors of a checkpoint do not fit the model: lists all that is missing,
    unexpected or of the wrong shape."""

    def __init__(self, where: str, missing: List[str], unexpected: List[str],
                 wrong: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]], bad_dtype: List[Tuple[str, str]]):
        self.missing, self.unexpected, self.wrong, self.bad_dtype = missing, unexpected, wrong, bad_dtype
        lines = [f"{where}: the tensors do not fit the model"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(exp)}" for n, got, exp in wrong))
        if bad_dtype:
            lines.append(f"  wrong dtype ({len(bad_dtype)}): " + ", ".join(f"{n} is {dt}" for n, dt in bad_dtype))
        super().__init__("\n".join(lines))


_FLOATS = (torch.float32, torch.bfloat16, torch.float16, torch.float64)
_INTS = (torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8)


def check_tensors(expected: Dict[str, TensorDecl], infos: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]], where: str) -> None:
    missing = [n for n, d in expected.items() if n not in infos and not d.optional]
    unexpected = [n for n in infos if n not in expected]
    wrong, bad = [], []
    for n, (dt, shape) in infos.items():
        if n not in expected:
            continue
        if tuple(shape) != tuple(expected[n].shape):
            wrong.append((n, tuple(shape), tuple(expected[n].shape)))
        ok = dt in _INTS if expected[n].role == "table" else dt in _FLOATS
        if not ok:
            bad.append((n, str(dt)))
    if missing or unexpected or wrong or bad:
        raise WeightError(where, sorted(missing), sorted(unexpected), sorted(wrong), sorted(bad))


def load_model_weights(model, folder: str) -> None:
    """Check every tensor of `folder` against what `model` declares, then load."""
    store = WeightStore(folder)
    try:
        expected = model.tensors()
        check_tensors(expected, {n: store.info(n) for n in store.names()}, folder)
        model.load(store.get)
    finally:
        store.close()
