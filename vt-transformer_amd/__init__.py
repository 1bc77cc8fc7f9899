"""A small, whole inference engine for one MI355X: from a model folder
(config.json, safetensors) to next-token logits and generated tokens.

    from vt_transformer_amd import Engine, SamplingParams
    eng = Engine("/path/to/model", dtype="bfloat16")
    tokens = eng.generate([[1, 2, 3]], SamplingParams(max_tokens=16))
"""
from . import config, parts  # noqa: F401  (registers the built-in architecture and parts)
from .config import ConfigError, load_config, register_architecture
from .engine import Engine, ModelRunner, SchedulerConfig, StepEntry, load_model, make_runner, random_model
from .sampling import SamplingParams
from .weights import WeightError, write_random_model

__version__ = "0.1.0"
__all__ = ["Engine", "SamplingParams", "SchedulerConfig", "ModelRunner", "StepEntry", "load_model", "make_runner",
           "random_model", "load_config", "register_architecture", "write_random_model", "ConfigError", "WeightError"]
