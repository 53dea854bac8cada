from .loader import (
    WeightsError,
    checkpoint_files,
    iterate_checkpoint,
    load_model_dir,
    load_params,
    storage_dtype,
)
from .random_init import random_checkpoint_tensors, random_params, write_random_model

__all__ = [
    "WeightsError",
    "checkpoint_files",
    "iterate_checkpoint",
    "load_model_dir",
    "load_params",
    "random_checkpoint_tensors",
    "random_params",
    "storage_dtype",
    "write_random_model",
]
