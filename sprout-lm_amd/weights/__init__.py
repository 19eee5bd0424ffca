from .checkpoint import Checkpoint
from .loader import TensorSpec, WeightError, load_named_tensors, target_dtype
from .random_init import random_tensors, write_model_folder
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Checkpoint", "TensorSpec", "WeightError", "load_named_tensors", "target_dtype", "random_tensors",
           "write_model_folder", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
