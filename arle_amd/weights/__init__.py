from .loader import Checkpoint, WeightsError, compare_with_expected, load_weights
from .random_init import random_weights, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["Checkpoint", "WeightsError", "compare_with_expected", "load_weights", "random_weights",
           "write_random_model", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
