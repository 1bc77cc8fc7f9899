from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import architectures, config_from_dict, load_config, register_architecture
from .qwen2 import Qwen2Config

register_architecture(Qwen2Config.architecture, Qwen2Config)

__all__ = ["ConfigError", "LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "ScheduleEntry",
           "architectures", "config_from_dict", "load_config", "register_architecture", "Qwen2Config"]
