from .loader import check_tensors, load_model, random_model
from .random_init import random_tensor, random_tensors, write_model_dir

__all__ = ["check_tensors", "load_model", "random_model", "random_tensor", "random_tensors",
           "write_model_dir"]
