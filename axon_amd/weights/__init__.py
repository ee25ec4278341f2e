from .loader import CheckpointSource, WeightError, WeightStore, check_tensors
from .random_init import RandomSource, write_random_model
from .safetensors_io import Checkpoint, SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["CheckpointSource", "WeightError", "WeightStore", "check_tensors", "RandomSource", "write_random_model",
           "Checkpoint", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
