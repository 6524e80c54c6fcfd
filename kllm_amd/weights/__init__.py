from .safetensors_io import (Checkpoint, SafetensorsError, SafetensorsFile, TensorEntry,
                             write_safetensors)
from .loader import WeightError, check_checkpoint, load_weights, merge_specs, target_dtype
from .random_init import random_tensor, random_weights, write_random_model

__all__ = [
    "Checkpoint", "SafetensorsError", "SafetensorsFile", "TensorEntry", "write_safetensors",
    "WeightError", "check_checkpoint", "load_weights", "merge_specs", "target_dtype",
    "random_tensor", "random_weights", "write_random_model",
]
