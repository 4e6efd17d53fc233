"""The step function, the scheduler above it, and generation."""

from .batch import StepContext, StepEntry, StepError, build_step  # noqa: F401
from .model import DecoderModel, require_gpu, run_dtype  # noqa: F401
from .runner import ModelRunner  # noqa: F401
from .scheduler import Request, ScheduledEntry, Scheduler  # noqa: F401
from .engine import Engine  # noqa: F401
