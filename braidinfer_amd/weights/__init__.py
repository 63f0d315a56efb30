from .safetensors_io import (SafetensorsFile, SafetensorsFolder, SafetensorsWriter, write_safetensors, plan_shards,
                             INDEX_NAME)
from .loader import (TensorSpec, FolderTensors, RandomTensors, WeightArena, LoadProfile, load_tensors,
                     write_model_folder, resident_bytes)
from .random_weights import random_tensor, random_tensors, tensor_key, normal_f32, ones_f32, f32_to_bf16_bits

__all__ = ["SafetensorsFile", "SafetensorsFolder", "SafetensorsWriter", "write_safetensors", "plan_shards", "INDEX_NAME",
           "TensorSpec", "FolderTensors", "RandomTensors", "WeightArena", "LoadProfile", "load_tensors",
           "write_model_folder", "resident_bytes", "random_tensor", "random_tensors", "tensor_key", "normal_f32",
           "ones_f32", "f32_to_bf16_bits"]
