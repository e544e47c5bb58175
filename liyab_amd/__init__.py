"""liyab_amd: a small, whole inference engine for one MI355X (gfx950)."""

from . import config as config  # noqa: F401  (registers the architectures)
from .errors import (  # noqa: F401
    Busy,
    ContextFull,
    InvalidArgument,
    InvalidModel,
    KernelError,
    LiyabError,
    OutOfPages,
    Unsupported,
)

__version__ = "0.1.0"
