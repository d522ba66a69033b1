from .contract import Contract, TensorSpec, WeightError
from .loader import WeightStore, compute_dtype, load_checkpoint, store_from_tensors
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, read_header, write_safetensors

__all__ = ["Contract", "TensorSpec", "WeightError", "WeightStore", "compute_dtype", "load_checkpoint",
           "store_from_tensors", "random_tensors", "write_random_model", "SafetensorsError",
           "read_header", "write_safetensors"]
