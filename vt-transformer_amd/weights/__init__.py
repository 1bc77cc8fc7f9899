from .safetensors_io import SafetensorsFile, WeightFileError, WeightStore, write_safetensors
from .loader import WeightError, check_tensors, load_model_weights
from .random_init import declared_tensors, random_tensor, random_tensors, write_random_model

__all__ = ["SafetensorsFile", "WeightFileError", "WeightStore", "write_safetensors", "WeightError", "check_tensors",
           "load_model_weights", "declared_tensors", "random_tensor", "random_tensors", "write_random_model"]
