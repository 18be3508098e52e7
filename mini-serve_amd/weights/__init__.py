from .loader import WeightsError, load_weights
from .random_init import Init, random_tensors, write_model_folder

__all__ = ["WeightsError", "load_weights", "Init", "random_tensors", "write_model_folder"]
