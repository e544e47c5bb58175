"""Step function, scheduler and generation."""

from .core import EngineCore  # noqa: F401
from .step import StepFunction, StepItem  # noqa: F401
