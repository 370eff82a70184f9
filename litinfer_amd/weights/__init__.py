from .safetensors_io import SafetensorsFile, write_safetensors
from .loader import (CheckpointFolder, ParamSpec, TensorSource, WeightError, check_entries, load_into,
                     stored_precision)
from .random_init import random_tensor, random_tensors, write_random_model

__all__ = ["SafetensorsFile", "write_safetensors", "CheckpointFolder", "ParamSpec", "TensorSource", "WeightError",
           "check_entries", "load_into", "stored_precision", "random_tensor", "random_tensors",
           "write_random_model"]
