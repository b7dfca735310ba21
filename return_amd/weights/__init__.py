from .loader import WeightError, load_weights
from .random_init import random_weights, write_model_folder

__all__ = ["WeightError", "load_weights", "random_weights", "write_model_folder"]
