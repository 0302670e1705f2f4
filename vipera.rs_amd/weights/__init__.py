from .checkpoint import INT_TABLE, MATRIX, VECTOR, Checkpoint, TensorSpec, WeightsError, kept_bytes, kept_dtype, load_tensors
from .random_init import (random_device_tensors, random_tensor, random_tensors, standard_normal, tensor_key,
                          write_random_model)
from .safetensors_io import SafetensorsFile, TensorInfo, write_safetensors

__all__ = [
    "INT_TABLE", "MATRIX", "VECTOR", "Checkpoint", "TensorSpec", "WeightsError", "kept_bytes", "kept_dtype",
    "load_tensors", "random_device_tensors", "random_tensor", "random_tensors", "standard_normal", "tensor_key",
    "write_random_model", "SafetensorsFile", "TensorInfo", "write_safetensors",
]
