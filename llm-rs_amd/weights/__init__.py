from .loader import WeightError, check_tensors, load_tensors, open_model_files, stored_dtype
from .random_init import RandomTensors, fill_normal, random_tensors, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["WeightError", "check_tensors", "load_tensors", "open_model_files", "stored_dtype",
           "RandomTensors", "fill_normal", "random_tensors", "write_model_folder", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
