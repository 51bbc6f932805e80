from .loader import WeightError, iter_tensors, load_state_dict, load_weights, weight_files
from .random_init import fill_random_, random_state_dict, write_random_model

__all__ = ["WeightError", "iter_tensors", "load_state_dict", "load_weights", "weight_files", "fill_random_",
           "random_state_dict", "write_random_model"]
