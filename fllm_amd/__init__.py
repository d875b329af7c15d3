"""fllm_amd: a Llama inference engine for one MI355X (gfx950)."""
from . import models as _models  # noqa: F401  (registers the architectures)
from . import parts as _parts    # noqa: F401  (registers the parts)

__version__ = "0.1.0"

from .engine import Engine, ModelRunner, StepEntry, TokenEvent  # noqa: E402
from .sampling import SamplingParams  # noqa: E402

__all__ = ["Engine", "ModelRunner", "StepEntry", "TokenEvent", "SamplingParams"]
