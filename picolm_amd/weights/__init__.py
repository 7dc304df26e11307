from .checkpoint import (Checkpoint, TensorDict, TensorSpec, WeightFetcher, WeightsError,
                         canonical_name, check_specs, stored_dtype)
from .random_init import RandomWeights, random_tensor, random_tensors, write_random_model
from .safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors

__all__ = [
    "Checkpoint", "TensorDict", "TensorSpec", "WeightFetcher", "WeightsError", "canonical_name",
    "check_specs", "stored_dtype", "RandomWeights", "random_tensor", "random_tensors",
    "write_random_model", "SafetensorsError", "SafetensorsFile", "write_safetensors",
]
