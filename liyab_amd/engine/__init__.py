"""Step function, scheduler and generation."""

from .core import EngineCore  # noqa: F401
from .engine import Engine, GenerationResult, GenerationStats  # noqa: F401
from .scheduler import Request, Scheduled, Scheduler, SchedulerStats  # noqa: F401
from .step import StepFunction, StepItem  # noqa: F401
