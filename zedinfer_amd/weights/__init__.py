from .loader import WeightError, WeightSpec, canonical_name, check_names, load_weights, storage_dtype
from .random_weights import random_weights, write_model_folder
from .safetensors_io import (SafetensorsError, SafetensorsFile, SafetensorsFolder,
                             write_safetensors)

__all__ = [
    "WeightError", "WeightSpec", "canonical_name", "check_names", "load_weights", "storage_dtype",
    "random_weights", "write_model_folder", "SafetensorsError", "SafetensorsFile",
    "SafetensorsFolder", "write_safetensors",
]
