from .spec import TensorSpec, MATRIX, VECTOR, TABLE, NORMAL, ONE_PLUS_NORMAL
from .loader import WeightError, load_model, read_tensors, resolve_dtype, shard_names
from .random_init import random_model, random_tensors, write_model_folder, draw_tensor

__all__ = ["TensorSpec", "MATRIX", "VECTOR", "TABLE", "NORMAL", "ONE_PLUS_NORMAL", "WeightError",
           "load_model", "read_tensors", "resolve_dtype", "shard_names", "random_model",
           "random_tensors", "write_model_folder", "draw_tensor"]
