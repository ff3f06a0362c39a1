from .safetensors_io import SafetensorsError, SafetensorsFile, TensorIndex, write_safetensors, write_state_dict
from .loader import WeightError, check_names, load_model_weights, load_state_dict
from .random_init import random_state, random_tensor, write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "TensorIndex", "write_safetensors", "write_state_dict",
           "WeightError", "check_names", "load_model_weights", "load_state_dict", "random_state",
           "random_tensor", "write_random_model"]
