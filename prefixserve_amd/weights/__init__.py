from .loader import WeightLoadError, load_weights, shard_files
from .random_init import random_tensors, write_random_model

__all__ = ["WeightLoadError", "load_weights", "random_tensors", "shard_files", "write_random_model"]
