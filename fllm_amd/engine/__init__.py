from .context import CacheBinding, StepContext
from .model import Model
from .runner import ModelRunner, StepEntry, StepError, parse_dtype

__all__ = ["CacheBinding", "StepContext", "Model", "ModelRunner", "StepEntry", "StepError", "parse_dtype"]
