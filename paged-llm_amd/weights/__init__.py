from .loader import WeightsError, load_state_dict, load_weights
from .random_init import fill_random, write_random_model

__all__ = ["WeightsError", "load_state_dict", "load_weights", "fill_random", "write_random_model"]
