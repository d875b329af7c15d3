from .context import CacheBinding, StepContext
from .model import Model
from .runner import ModelRunner, StepEntry, StepError, parse_dtype

__all__ = ["CacheBinding", "StepContext", "Model", "ModelRunner", "StepEntry", "StepError", "parse_dtype"]
from .engine import Engine, EngineStats, TokenEvent  # noqa: E402
from .scheduler import ScheduledStep, Scheduler, SchedulerConfig, Sequence  # noqa: E402

__all__ += ["Engine", "EngineStats", "TokenEvent", "ScheduledStep", "Scheduler", "SchedulerConfig", "Sequence"]
