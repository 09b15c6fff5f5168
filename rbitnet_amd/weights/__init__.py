from .safetensors_io import SafetensorsFile, WeightFolder, save_file
from .loader import load_weights, resolve_names
from .random_init import write_random_model, random_tensors, random_tensor, RandomTensors, DEFAULT_SEED

__all__ = ["SafetensorsFile", "WeightFolder", "save_file", "load_weights", "resolve_names",
           "write_random_model", "random_tensors", "random_tensor", "RandomTensors", "DEFAULT_SEED"]
