from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (register the parts)
from .base import Block, FeedForward, KVNeed, Mixer, Norm, Part, StateNeed
from .runtime import Runtime

__all__ = ["Block", "FeedForward", "KVNeed", "Mixer", "Norm", "Part", "StateNeed", "Runtime"]
