from .loader import LoadedModel, WeightsError, fit_tensors, load_model_folder, read_config, run_dtype
from .random_init import random_model, random_tensor, random_tensors, write_model_folder

__all__ = [
    "LoadedModel",
    "WeightsError",
    "fit_tensors",
    "load_model_folder",
    "random_model",
    "random_tensor",
    "random_tensors",
    "read_config",
    "run_dtype",
    "write_model_folder",
]
