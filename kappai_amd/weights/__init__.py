from .loader import WeightsError, check_and_load, parse_dtype, stored_to_runtime
from .random_init import random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .spec import (INIT_NORMAL, INIT_ONES, INIT_SMALL, MATRIX, TABLE, VECTOR, TensorSpec)

__all__ = ["WeightsError", "check_and_load", "parse_dtype", "stored_to_runtime", "random_tensor",
           "random_tensors", "write_random_model", "SafetensorsError", "SafetensorsFile",
           "write_safetensors", "INIT_NORMAL", "INIT_ONES", "INIT_SMALL", "MATRIX", "TABLE",
           "VECTOR", "TensorSpec"]
