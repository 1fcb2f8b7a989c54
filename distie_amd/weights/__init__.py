from .loader import (WeightsError, check_names, kept_dtype, load_into, random_into,
                     write_random_model)
from .safetensors_io import SafetensorsError, SafetensorsFile, model_files, write_safetensors

__all__ = ["WeightsError", "check_names", "kept_dtype", "load_into", "random_into", "write_random_model",
           "SafetensorsError", "SafetensorsFile", "model_files", "write_safetensors"]
