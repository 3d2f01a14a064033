from tokensprint_amd.weights.loader import (
    CheckpointFiles, TensorDict, WeightsError, check_tensors, held_dtype, load_weights,
)
from tokensprint_amd.weights.random_init import (
    declared_tensors, random_tensors, write_random_model,
)

__all__ = ["CheckpointFiles", "TensorDict", "WeightsError", "check_tensors", "held_dtype",
           "load_weights", "declared_tensors", "random_tensors", "write_random_model"]
