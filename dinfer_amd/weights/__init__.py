from .loader import WeightError, WeightLoader
from .random_init import write_random_model
from .safetensors_io import SafetensorsDir, WeightFileError, write_safetensors

__all__ = ["WeightError", "WeightLoader", "write_random_model", "SafetensorsDir", "WeightFileError",
           "write_safetensors"]
