"""Weights: needs of a model, safetensors reading, seeded random weights."""
from .needs import TensorNeed
from .store import read_tensor, read_tensors, shard_files
from .random_init import random_tensor, random_tensors, write_model_folder

__all__ = ["TensorNeed", "read_tensor", "read_tensors", "shard_files", "random_tensor", "random_tensors",
           "write_model_folder"]
