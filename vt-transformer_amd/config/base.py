"""Typed description of a model, independent of any one architecture.

An architecture's configuration class (for instance ``Qwen2Config``) reads the
keys of its own ``config.json`` and turns them into a :class:`ModelSpec`: a
list of layers, each naming the kind and the constants of its mixer,
feed-forward, norms and position encoding, plus the order in which the layers
run.  Everything below the configuration (weights, parts, cache manager, step
function) works from the ``ModelSpec`` alone and never asks which
architecture it came from.

The reference keeps these constants at the head of each model program
(v1/models/qwen2-7b/inference_fp16.dag:1-15) and copies them by hand into C++
(v1/models/qwen2-7b/memory.hpp:3-7); here they are read once from
``config.json``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """A config.json that cannot be used: a missing key, a wrong type, an
    option that this engine does not implement."""


@dataclass(frozen=True)
class PartSpec:
    """Kind and constants of one part.  ``kind`` is looked up in the part
    registry of its role; ``params`` are passed to the part's constructor."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def key(self) -> str:
        return self.kind + ":" + json.dumps(self.params, sort_keys=True, default=str)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: how its parts are arranged (``block``), and the parts."""

    block: PartSpec
    mixer: PartSpec
    feed_forward: PartSpec
    norms: Dict[str, PartSpec]
    prefix: str  # tensor-name prefix of this layer, e.g. "model.layers.3."


@dataclass(frozen=True)
class ScheduleEntry:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named twice: its
    weights are shared, each entry still has a cache of its own).
    ``cache_from`` names an earlier entry of the schedule whose cache this
    entry reads instead of writing its own (None: own cache)."""

    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    head: PartSpec
    max_positions: int
    eos_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None

    def validate(self) -> None:
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ConfigError(f"schedule[{i}] names layer {e.layer}, model has {n} layers")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ConfigError(
                        f"schedule[{i}] reads the cache of entry {e.cache_from}, which does not run before it")
                if self.schedule[e.cache_from].cache_from is not None:
                    raise ConfigError(
                        f"schedule[{i}] reads the cache of entry {e.cache_from}, which has no cache of its own")


class ModelConfig:
    """Base class of an architecture's typed configuration.

    Subclasses are dataclasses with the architecture's own fields, a
    ``from_dict`` that reads its config.json keys, ``to_dict`` that writes
    them back, and ``to_spec``."""

    architecture: str = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError

    def to_spec(self) -> ModelSpec:
        raise NotImplementedError

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(self.to_dict(), f, indent=2)


# ---------------------------------------------------------------------------
# helpers for reading config.json keys with one clear error each
# ---------------------------------------------------------------------------

_MISSING = object()


def read_key(d: Dict[str, Any], key: str, typ, default=_MISSING, *, where: str = "config.json"):
    if key not in d or d[key] is None:
        if default is _MISSING:
            raise ConfigError(f"{where}: required key '{key}' is missing")
        return default
    v = d[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, float) and v == int(v):
        v = int(v)
    if typ is int and isinstance(v, bool):
        raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
    if not isinstance(v, typ):
        raise ConfigError(f"{where}: key '{key}' must be {typ.__name__}, got {v!r}")
    return v


def require_positive(name: str, v) -> None:
    if not v > 0:
        raise ConfigError(f"config.json: '{name}' must be positive, got {v!r}")
