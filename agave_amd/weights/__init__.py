"""Weights: the safetensors container, checked loading by name, random-weights mode."""
from .loader import DictWeightSource, TensorNeed, WeightError, WeightSource, check_tensors
from .random_init import RandomWeightSource, random_tensors, write_random_model
from .safetensors_io import Checkpoint, SafetensorsError, write_safetensors

__all__ = ["Checkpoint", "SafetensorsError", "write_safetensors", "TensorNeed", "WeightError",
           "WeightSource", "DictWeightSource", "check_tensors", "random_tensors", "write_random_model", "RandomWeightSource"]
