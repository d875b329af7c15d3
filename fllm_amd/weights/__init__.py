from .loader import WeightsError, check_tensors, expected_tensors, load_checkpoint, part_weights
from .random_init import random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, open_checkpoint, write_safetensors

__all__ = ["WeightsError", "check_tensors", "expected_tensors", "load_checkpoint", "part_weights", "random_tensors",
           "write_random_model", "SafetensorsError", "SafetensorsFile", "open_checkpoint", "write_safetensors"]
