from .loader import WeightsError, held_dtype, load_tensors
from .random_init import InitRecipe, random_tensor, random_tensors, write_random_model

__all__ = ["InitRecipe", "WeightsError", "held_dtype", "load_tensors", "random_tensor", "random_tensors",
           "write_random_model"]
