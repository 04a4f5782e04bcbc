from .safetensors_io import SafetensorsError, SafetensorsFile, find_weight_files, write_safetensors
from .store import (DictSource, SafetensorsSource, TensorSpec, WeightError, WeightLoader, check, storage_dtype)
from .random_init import RandomSource, make_tensor, write_model_folder

__all__ = ["SafetensorsError", "SafetensorsFile", "find_weight_files", "write_safetensors", "DictSource",
           "SafetensorsSource", "TensorSpec", "WeightError", "WeightLoader", "check", "storage_dtype",
           "RandomSource", "make_tensor", "write_model_folder"]
