"""Sampling options of a request, with the reference's names, meanings and defaults
(rust/engine/src/sampling.rs:6-87)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

GREEDY_TEMPERATURE = 1e-5     # temperature at or below this takes the largest logit (sampling.rs:97-110)
_SEED_BASE = 0x8A5CD789635D2DFF
_SEED_STEP = 0x9E3779B97F4A7C15
_MASK64 = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0          # 0: greedy
    top_p: float = 1.0                # nucleus; 1: off
    top_k: int = 0                    # 0: off
    seed: Optional[int] = None        # Philox key; None: derived from the sequence id
    max_tokens: int = 16              # generated tokens at most
    stop_token_ids: Tuple[int, ...] = ()
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0.0:
            raise ValueError("temperature must be nonnegative")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError("top_p must be in [0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k must be nonnegative")
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        object.__setattr__(self, "stop_token_ids", tuple(int(t) for t in self.stop_token_ids))

    @property
    def greedy(self) -> bool:
        return self.temperature <= GREEDY_TEMPERATURE

    def stops_on(self, token: int, eos: Sequence[int]) -> bool:
        """Explicit stop ids always stop; end-of-sequence ids unless ignored (sampling.rs:89-93)."""
        return token in self.stop_token_ids or (not self.ignore_eos and token in eos)

    def seed_for(self, sequence_id: int) -> int:
        """sampling.rs:193-199: the request's seed, else one derived from the sequence id."""
        if self.seed is not None:
            return int(self.seed) & _MASK64
        return (_SEED_BASE ^ ((sequence_id * _SEED_STEP) & _MASK64)) & _MASK64
