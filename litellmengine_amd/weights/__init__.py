from .loader import WeightError, check_against, checkpoint_header, load_checkpoint, storage_dtype
from .random_init import random_tensor, random_weights, write_model_dir
from .spec import INIT_NORM, INIT_NORMAL, TensorSpec

__all__ = [
    "INIT_NORM",
    "INIT_NORMAL",
    "TensorSpec",
    "WeightError",
    "check_against",
    "checkpoint_header",
    "load_checkpoint",
    "random_tensor",
    "random_weights",
    "storage_dtype",
    "write_model_dir",
]
