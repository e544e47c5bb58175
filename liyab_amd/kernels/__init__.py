"""Hand-written HIP kernels for gfx950, as Python functions."""

from . import ops  # noqa: F401
from .lib import library_path, load  # noqa: F401
