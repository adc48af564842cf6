from .loader import TensorRule, check_names_and_shapes, load_weights
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafeTensorFile, write_safetensors

__all__ = ["SafeTensorFile", "TensorRule", "check_names_and_shapes", "load_weights",
           "random_tensors", "write_random_model", "write_safetensors"]
