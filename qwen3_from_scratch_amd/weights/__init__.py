from .checkpoint import Checkpoint, TensorSource, WeightError, check_tensors
from .random_init import RandomWeights, write_random_model

__all__ = [
    "Checkpoint",
    "TensorSource",
    "WeightError",
    "check_tensors",
    "RandomWeights",
    "write_random_model",
]
