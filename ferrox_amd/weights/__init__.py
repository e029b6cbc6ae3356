from .loader import CheckpointError, UnexpectedTensorsWarning, check_names, resident_dtype, upload
from .random_init import RandomSource, random_tensor
from .safetensors_io import Checkpoint, LazyTensor, SafetensorsError, SafetensorsFile, write_safetensors

__all__ = ["CheckpointError", "UnexpectedTensorsWarning", "check_names", "resident_dtype", "upload", "RandomSource", "random_tensor",
           "Checkpoint", "LazyTensor", "SafetensorsError", "SafetensorsFile", "write_safetensors"]
