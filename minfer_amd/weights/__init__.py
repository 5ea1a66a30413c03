from .loader import FolderWeights, TensorSpec, WeightError, check_against, storage_dtype
from .random_init import random_tensor, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_model_files, write_safetensors

__all__ = ["FolderWeights", "TensorSpec", "WeightError", "check_against", "storage_dtype",
           "random_tensor", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "open_model_files", "write_safetensors"]
