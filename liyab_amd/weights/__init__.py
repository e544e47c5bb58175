"""Weights: safetensors by tensor name, and the random-weights mode."""

from .loader import WEIGHTS_FILE, WeightStore  # noqa: F401
from .random_init import random_tensors, write_random_model  # noqa: F401
from .safetensors_io import SafetensorsFile, write_safetensors  # noqa: F401
