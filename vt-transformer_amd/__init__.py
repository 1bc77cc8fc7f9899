"""A small, whole inference engine for one MI355X: from a model folder
(config.json, safetensors) to next-token logits and generated tokens."""
from . import config, parts  # noqa: F401  (registers the built-in architecture and parts)

__version__ = "0.1.0"
