from .loader import TensorWant, WeightsError, check_names, kept_dtype, load_named_tensors
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors

__all__ = ["TensorWant", "WeightsError", "check_names", "kept_dtype", "load_named_tensors",
           "random_tensor", "random_tensors", "write_random_model",
           "SafetensorsError", "SafetensorsFile", "open_model_files", "write_safetensors"]
