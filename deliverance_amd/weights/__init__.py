from .safetensors_io import SafetensorsFile, WeightFileError, WeightSource, write_safetensors
from .loader import TensorDecl, WeightError, draw_tensor, load_declared, write_random_model

__all__ = ["SafetensorsFile", "WeightFileError", "WeightSource", "write_safetensors", "TensorDecl",
           "WeightError", "draw_tensor", "load_declared", "write_random_model"]
