from .loader import (TensorDecl, WeightError, load_tensors, random_tensor, random_tensors,
                     unique_decls, write_model_folder)
from .safetensors_io import Checkpoint, SafetensorsFile, WeightFileError, write_safetensors

__all__ = ["TensorDecl", "WeightError", "load_tensors", "random_tensor", "random_tensors",
           "unique_decls", "write_model_folder", "Checkpoint", "SafetensorsFile",
           "WeightFileError", "write_safetensors"]
