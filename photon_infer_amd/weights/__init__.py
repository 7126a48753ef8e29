from .loader import TensorSpec, check_tensors, load_model_tensors, storage_dtype
from .random_init import random_model_folder, random_tensors, write_random_model
from .safetensors_io import SafetensorsFile, open_model_files, write_safetensors

__all__ = ["TensorSpec", "check_tensors", "load_model_tensors", "storage_dtype", "random_tensors",
           "write_random_model", "random_model_folder", "SafetensorsFile", "open_model_files", "write_safetensors"]
