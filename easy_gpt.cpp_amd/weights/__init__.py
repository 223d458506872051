from .loader import CheckedWeights, WeightsError, check_names_and_shapes
from .random_init import RandomWeights, random_tensor, random_tensors, register_role, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = [
    "CheckedWeights", "RandomWeights", "SafetensorsError", "SafetensorsFile", "WeightsError", "check_names_and_shapes",
    "random_tensor", "random_tensors", "register_role", "write_random_model", "write_safetensors",
]
