from .loader import WeightError, check_names, load_weights, shard_files
from .random_init import random_tensor, random_tensors, write_model_folder

__all__ = [
    "WeightError",
    "check_names",
    "load_weights",
    "random_tensor",
    "random_tensors",
    "shard_files",
    "write_model_folder",
]
