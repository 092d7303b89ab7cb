from .loader import Checkpoint, UnexpectedTensors, WeightsError, compare_with_expected, load_weights
from .random_init import random_weights, register_init, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Checkpoint", "UnexpectedTensors", "WeightsError", "compare_with_expected", "load_weights", "random_weights",
           "register_init", "write_random_model", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
