from .loader import WeightsError, load_weights, weight_files
from .random_init import init_random, random_tensors, write_random_model

__all__ = ["WeightsError", "load_weights", "weight_files", "init_random", "random_tensors", "write_random_model"]
