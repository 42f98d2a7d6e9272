from .loader import ParamSpec, WeightsError, match_parameters, read_tensors
from .random_init import random_parameters, random_tensor, write_model_folder

__all__ = ["ParamSpec", "WeightsError", "match_parameters", "read_tensors", "random_parameters",
           "random_tensor", "write_model_folder"]
