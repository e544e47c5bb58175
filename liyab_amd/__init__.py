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

from .sampling import SamplingParams  # noqa: F401

__version__ = "0.1.0"


def __getattr__(name):
    # the engine needs torch and the GPU library: import it on first use
    if name in ("Engine", "EngineCore", "StepItem", "GenerationResult", "GenerationStats"):
        from . import engine

        return getattr(engine, name)
    raise AttributeError(name)
