from .safetensors_io import SafeTensorsFile, WeightError, write_safetensors
from .source import CheckpointSource, RandomSource, TensorSpec, check_tensors

__all__ = ["SafeTensorsFile", "WeightError", "write_safetensors", "CheckpointSource",
           "RandomSource", "TensorSpec", "check_tensors"]
