from kvforge_amd.weights.io import (WeightsError, read_safetensors_folder, read_tensors,
                                    tensor_index, write_safetensors)
from kvforge_amd.weights.loader import check_index, load_model_weights, runtime_dtype
from kvforge_amd.weights.random_init import random_tensors, write_random_model

__all__ = ["WeightsError", "read_safetensors_folder", "read_tensors", "tensor_index",
           "write_safetensors", "check_index", "load_model_weights", "runtime_dtype",
           "random_tensors", "write_random_model"]
