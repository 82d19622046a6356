from .safetensors_io import SafetensorsFile, SafetensorsError, write_safetensors
from .loader import Checkpoint, WeightsError, check_checkpoint, load_into
from .random_init import random_weights, write_random_model

__all__ = ["SafetensorsFile", "SafetensorsError", "write_safetensors", "Checkpoint", "WeightsError",
           "check_checkpoint", "load_into", "random_weights", "write_random_model"]
