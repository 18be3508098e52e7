from .loader import WeightsError, load_weights, tied_names
from .random_init import Init, random_tensors, write_model_folder

__all__ = ["WeightsError", "load_weights", "tied_names", "Init", "random_tensors", "write_model_folder"]
