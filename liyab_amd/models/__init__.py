"""The generic decoder and model loading."""

from .decoder import DecoderModel  # noqa: F401
from .loading import load_model, resolve_dtype  # noqa: F401
