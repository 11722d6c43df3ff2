from .loader import TensorSpec, WeightError, load_tensors, match_specs, storage_dtype
from .safetensors_io import ModelFiles, SafetensorsFile, save_safetensors, SafetensorsError
from .random_init import write_random_model, random_tensors, random_tensor

__all__ = ["TensorSpec", "WeightError", "load_tensors", "match_specs", "storage_dtype", "ModelFiles",
           "SafetensorsFile", "save_safetensors", "SafetensorsError", "write_random_model",
           "random_tensors", "random_tensor"]
