from .loader import TensorDecl, WeightError, check_names, load_tensors, storage_dtype
from .random_init import random_tensors, random_tensors_on_device, write_random_model
from .safetensors_io import (SafetensorsError, SafetensorsFile, checkpoint_files,
                             read_header, write_file)

__all__ = [
    "TensorDecl", "WeightError", "check_names", "load_tensors", "storage_dtype",
    "random_tensors", "random_tensors_on_device", "write_random_model", "SafetensorsError", "SafetensorsFile",
    "checkpoint_files", "read_header", "write_file",
]
