"""Reading and writing safetensors files by tensor name.

Format as the reference reads it (vt-transformer/core/safetensors.hpp:159-201):
8 bytes little-endian header length, a JSON header mapping each tensor name
to {dtype, shape, data_offsets} with offsets relative to the end of the
header, then the raw data.  A folder may instead hold
`model.safetensors.index.json` whose `weight_map` names the shard of each
tensor (safetensors.hpp:204-267).

Tensors are memory-mapped, not read: a 145 GB checkpoint is never held in
host memory as a whole.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import numpy as np
import torch


class WeightFileError(IOError):
    pass


_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsFile:
    def __init__(self, path: str):
        self.path = path
        try:
            size = os.path.getsize(path)
            self._f = open(path, "rb")
        except OSError as e:
            raise WeightFileError(f"{path}: cannot open ({e.strerror})") from None
        if size < 8:
            raise WeightFileError(f"{path}: truncated (shorter than its 8-byte header length)")
        (hlen,) = struct.unpack("<Q", self._f.read(8))
        if 8 + hlen > size:
            raise WeightFileError(f"{path}: truncated (header of {hlen} bytes does not fit in {size} bytes)")
        try:
            header = json.loads(self._f.read(hlen).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not valid JSON ({e})") from None
        self._data_start = 8 + hlen
        self._size = size
        self.metadata = header.pop("__metadata__", {}) or {}
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            dt = e.get("dtype")
            if dt not in _DTYPES:
                raise WeightFileError(f"{path}: tensor '{name}' has unknown dtype {dt!r}")
            tdt, isz = _DTYPES[dt]
            shape = tuple(int(s) for s in e["shape"])
            b, en = (int(x) for x in e["data_offsets"])
            n = 1
            for s in shape:
                n *= s
            if en - b != n * isz:
                raise WeightFileError(
                    f"{path}: tensor '{name}' of shape {list(shape)} {dt} needs {n * isz} bytes, file gives {en - b}")
            if self._data_start + en > size:
                raise WeightFileError(f"{path}: truncated (tensor '{name}' ends beyond the file)")
            self.entries[name] = (tdt, shape, b, en)
        self._mm = None

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        e = self.entries[name]
        return e[0], e[1]

    def get(self, name: str) -> torch.Tensor:
        """The tensor as a read-only view of the mapped file (CPU)."""
        tdt, shape, b, en = self.entries[name]
        if self._mm is None:
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        if en == b:
            return torch.empty(shape, dtype=tdt)
        raw = np.frombuffer(self._mm, dtype=np.uint8, count=en - b, offset=self._data_start + b)
        with _quiet_readonly():
            t = torch.from_numpy(raw)
        return t.view(tdt).reshape(shape)

    def close(self) -> None:
        self._mm = None
        self._f.close()


class _quiet_readonly:
    """torch warns when it wraps a read-only numpy array; the views made
    here are only ever copied from."""

    def __enter__(self):
        import warnings
        self._cm = warnings.catch_warnings()
        self._cm.__enter__()
        warnings.simplefilter("ignore")

    def __exit__(self, *a):
        return self._cm.__exit__(*a)


class WeightStore:
    """All tensors of a model folder by name, over one file or shards."""

    def __init__(self, folder: str):
        self.folder = folder
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, "model.safetensors.index.json")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.isfile(single):
            f = SafetensorsFile(single)
            self._files[single] = f
            for n in f.names():
                self._where[n] = single
        elif os.path.isfile(index):
            with open(index) as fh:
                try:
                    wm = json.load(fh)["weight_map"]
                except (json.JSONDecodeError, KeyError, TypeError) as e:
                    raise WeightFileError(f"{index}: no usable 'weight_map' ({e})") from None
            for shard in sorted(set(wm.values())):
                p = os.path.join(folder, shard)
                f = SafetensorsFile(p)
                self._files[p] = f
                for n in f.names():
                    if n in self._where:
                        raise WeightFileError(f"{p}: tensor '{n}' is also in {self._where[n]}")
                    self._where[n] = p
        else:
            raise WeightFileError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def info(self, name: str):
        return self._files[self._where[name]].info(name)

    def get(self, name: str) -> torch.Tensor:
        return self._files[self._where[name]].get(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write `tensors` (name, CPU tensor) to `path`, one tensor at a time."""
    items = [(n, t.detach().contiguous()) for n, t in tensors]
    header = {}
    off = 0
    for n, t in items:
        if t.dtype not in _NAMES:
            raise WeightFileError(f"cannot store tensor '{n}' of dtype {t.dtype}")
        nbytes = t.numel() * t.element_size()
        header[n] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + nbytes]}
        off += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    hb = json.dumps(header, separators=(",", ":")).encode("utf-8")
    hb += b" " * ((8 - len(hb) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hb)))
        f.write(hb)
        for n, t in items:
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
