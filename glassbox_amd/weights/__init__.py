from .loader import (WeightError, build_model, compute_dtype, init_random, load_model, load_weights,
                     random_tensors, write_random_model)
from .safetensors_io import SafetensorsFile, save_file

__all__ = ["WeightError", "build_model", "compute_dtype", "init_random", "load_model", "load_weights",
           "random_tensors", "write_random_model", "SafetensorsFile", "save_file"]
