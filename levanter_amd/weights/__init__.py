from .loader import WeightsError, load_tensors
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, save_file

__all__ = ["WeightsError", "load_tensors", "random_tensors", "write_random_model", "SafetensorsError",
           "SafetensorsFile", "open_model_files", "save_file"]
