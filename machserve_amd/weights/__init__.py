from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors
from .checkpoint import Checkpoint, TensorDict
from .loader import WeightsError, load_weights
from .random_init import random_tensor_dict, random_tensors, write_random_model

__all__ = ["SafetensorsError", "SafetensorsFile", "write_safetensors", "Checkpoint", "TensorDict", "WeightsError",
           "load_weights", "random_tensor_dict", "random_tensors", "write_random_model"]
