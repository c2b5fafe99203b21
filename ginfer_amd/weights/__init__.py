from .safetensors_file import SafetensorsFile, SafetensorsError, write_safetensors, open_model_files
from .loader import WeightSpec, WeightError, load_weights, check_against
from .random_init import write_random_model, bind_random_weights

__all__ = ["SafetensorsFile", "SafetensorsError", "write_safetensors", "open_model_files",
           "WeightSpec", "WeightError", "load_weights", "check_against", "write_random_model", "bind_random_weights"]
