from .loader import (Source, WeightError, build_model, checkpoint_layout, checkpoint_tensors, compute_dtype, init_random,
                     load_model, load_weights, random_tensors, write_random_model)
from .safetensors_io import SafetensorsFile, save_file

__all__ = ["Source", "checkpoint_layout", "checkpoint_tensors", "WeightError", "build_model", "compute_dtype", "init_random", "load_model", "load_weights",
           "random_tensors", "write_random_model", "SafetensorsFile", "save_file"]
