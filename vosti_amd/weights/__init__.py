from .loader import WeightError, load_weights, open_checkpoint
from .random_init import random_tensor_cpu, random_weights_on_gpu, write_random_model

__all__ = ["WeightError", "load_weights", "open_checkpoint", "random_tensor_cpu", "random_weights_on_gpu",
           "write_random_model"]
