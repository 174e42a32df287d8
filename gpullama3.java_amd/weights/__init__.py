from .loader import TensorSpec, WeightsError, kept_dtype, load_weights, weight_files
from .random_init import random_tensor, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["TensorSpec", "WeightsError", "kept_dtype", "load_weights", "weight_files", "random_tensor",
           "write_random_model", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
