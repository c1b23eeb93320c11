from .loader import WeightError, check, load_folder, target_dtype
from .random_init import random_tensor, random_tensors, write_model_folder
from .safetensors_io import SafetensorsFile, WeightFileError, open_folder, write_file

__all__ = ["WeightError", "check", "load_folder", "target_dtype", "random_tensor", "random_tensors",
           "write_model_folder", "SafetensorsFile", "WeightFileError", "open_folder", "write_file"]
