from .loader import WeightError, ShardSet, load_tensors
from .random_init import random_tensors, write_model_dir
from .spec import INT_TABLE, MATRIX, VECTOR, TensorSpec

__all__ = ["WeightError", "load_tensors", "ShardSet", "random_tensors", "write_model_dir", "TensorSpec",
           "MATRIX", "VECTOR", "INT_TABLE"]
