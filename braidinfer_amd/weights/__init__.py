from .safetensors_io import SafetensorsFile, SafetensorsFolder, write_safetensors
from .loader import TensorSpec, load_tensors, random_tensors, write_model_folder

__all__ = ["SafetensorsFile", "SafetensorsFolder", "write_safetensors", "TensorSpec", "load_tensors",
           "random_tensors", "write_model_folder"]
