from .loader import CheckpointFiles, ParamDecl, check_declared, load_weights
from .random_init import random_tensor, write_random_model
from .safetensors_io import SafetensorsFile, write_safetensors

__all__ = ["CheckpointFiles", "ParamDecl", "check_declared", "load_weights", "random_tensor", "write_random_model",
           "SafetensorsFile", "write_safetensors"]
