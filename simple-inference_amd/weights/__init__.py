from .loader import WeightError, check_names_and_shapes, load_weights, target_dtype
from .random_init import random_tensors, write_model_folder

__all__ = ["WeightError", "check_names_and_shapes", "load_weights", "target_dtype",
           "random_tensors", "write_model_folder"]
