from .loader import WeightError, expand_weight_map, load_state_dict, load_weights
from .random_init import fill_random, write_random_model
from .safetensors_io import ModelFiles, SafetensorsError, SafetensorsFile, SafetensorsWriter, save_file

__all__ = [
    "ModelFiles", "SafetensorsError", "SafetensorsFile", "SafetensorsWriter", "WeightError",
    "expand_weight_map", "fill_random", "load_state_dict", "load_weights", "save_file", "write_random_model",
]
