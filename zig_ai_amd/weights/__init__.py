"""Weights: safetensors I/O, loading by name, and random model folders."""

from .safetensors_io import Checkpoint, SafetensorsError, SafetensorsFile, write_safetensors  # noqa: F401
from .loader import WeightError, expected_tensors, keep_dtype, load_tensors  # noqa: F401
from .random_init import random_tensors, write_random_model  # noqa: F401
