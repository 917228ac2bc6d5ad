from .loader import WeightsError, load_model
from .random_init import random_model_on_device, write_random_model
from .safetensors_io import SafetensorsFile, write_safetensors

__all__ = ["WeightsError", "load_model", "random_model_on_device", "write_random_model", "SafetensorsFile",
           "write_safetensors"]
