from .loader import WeightsError, load_state, load_weights, open_folder
from .random_weights import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["WeightsError", "load_state", "load_weights", "open_folder", "random_tensors", "write_random_model",
           "SafetensorsError", "SafetensorsFile", "write_safetensors"]
