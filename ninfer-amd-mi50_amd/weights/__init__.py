from .safetensors_io import SafeTensorsFile, WeightError, write_safetensors
from . import counter_random
from .source import CheckpointSource, RandomSource, TensorSpec, check_tensors

__all__ = ["SafeTensorsFile", "WeightError", "write_safetensors", "CheckpointSource",
           "RandomSource", "counter_random", "TensorSpec", "check_tensors"]
