from .loader import WeightsError, load_tensors, target_dtype
from .random_init import random_tensors, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors

__all__ = ["WeightsError", "load_tensors", "target_dtype", "random_tensors", "write_model_folder",
           "SafetensorsError", "SafetensorsFile", "open_model_files", "write_safetensors"]
