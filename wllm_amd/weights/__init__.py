from wllm_amd.weights.checkpoint import Checkpoint, ExpectedTensor, TensorFetcher, WeightError
from wllm_amd.weights.random_init import random_tensor, write_random_model
from wllm_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = [
    "Checkpoint", "ExpectedTensor", "TensorFetcher", "WeightError", "random_tensor",
    "write_random_model", "SafetensorsError", "SafetensorsFile", "write_safetensors",
]
