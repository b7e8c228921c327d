from .loader import WeightsError, check_names, load_weights, stored_dtype
from .random_init import RandomInit, build_model, random_model_on_device, random_tensor, write_random_model
from .reader import CheckpointReader

__all__ = ["WeightsError", "check_names", "load_weights", "stored_dtype", "RandomInit", "build_model",
           "random_model_on_device", "random_tensor", "write_random_model", "CheckpointReader"]
