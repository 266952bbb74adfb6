from .loader import WeightError, kept_dtype, load_weights
from .random_init import random_tensors, write_random_model

__all__ = ["WeightError", "kept_dtype", "load_weights", "random_tensors", "write_random_model"]
