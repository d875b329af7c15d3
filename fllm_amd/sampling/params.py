"""Sampling options of a request, with the reference's names, meanings and defaults
(rust/engine/src/sampling.rs:6-87)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

GREEDY_TEMPERATURE = 1e-5     # temperature at or below this takes the largest logit (sampling.rs:97-110)
_SEED_BASE = 0x8A5CD789635D2DFF
_SEED_STEP = 0x9E3779B97F4A7C15
_MASK64 = (1 << 64) - 1
MAX_CHOICES = 16              # answers to one prompt at most (rust/engine/src/runtime.rs:399-401)
_CHOICE_SEED_STEP = 0x9E3779B97F4A7C15
MAX_TOP_LOGPROBS = 20         # alternatives a token at most (sampling.rs:950)


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0          # 0: greedy
    top_p: float = 1.0                # nucleus; 1: off
    top_k: int = 0                    # 0: off
    seed: Optional[int] = None        # Philox key; None: derived from the sequence id
    max_tokens: int = 16              # generated tokens at most
    stop_token_ids: Tuple[int, ...] = ()
    ignore_eos: bool = False
    min_p: float = 0.0                # drops what weighs less than min_p times the likeliest token; 0: off
    repetition_penalty: float = 1.0   # logits of tokens seen before: divided by it when positive, multiplied otherwise; 1: off
    presence_penalty: float = 0.0     # taken off the logit of every token seen before
    frequency_penalty: float = 0.0    # taken off once for every time the token was seen
    repeat_last_n: int = -1           # tokens of the history (prompt and generated) the penalties look at; negative: all
    logit_bias: Tuple[Tuple[int, float], ...] = ()   # (token id, what is added to its logit)
    min_tokens: int = 0               # no end-of-sequence or stop id before this many tokens were generated
    priority: int = 0                 # smaller values are served first under the `priority` scheduling policy
    n: int = 1                        # answers to the one prompt (the reference's `choices`): each with draws of its own
    allowed_token_ids: Tuple[int, ...] = ()          # when not empty, only these tokens can be chosen
    bad_word_ids: Tuple[Tuple[int, ...], ...] = ()   # token sequences that must not appear: the last token of one cannot
                                                     # be chosen once the tokens before it stand at the end of the history
    timeout_secs: Optional[float] = None             # the request is given up this long after it was added (waiting included)
    logprobs: Optional[int] = None    # None: off; n: every token comes with its log-probability in the model's own
                                      # distribution (before penalties, temperature and filters) and the n likeliest tokens
    logprobs_processed: bool = False  # the reference's `logprobs_mode: processed_logprobs`: the log-probabilities are those
                                      # of the distribution the token was drawn from (after penalties, temperature and
                                      # filters; greedy: a point mass), the alternatives the likeliest tokens that are left

    def __post_init__(self):
        if self.temperature < 0.0:
            raise ValueError("temperature must be nonnegative")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError("top_p must be in [0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k must be nonnegative")
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError("min_p must be in [0, 1]")
        if not self.repetition_penalty > 0.0:
            raise ValueError("repetition_penalty must be positive")
        if self.min_tokens < 0:
            raise ValueError("min_tokens must be nonnegative")
        if not 1 <= int(self.n) <= MAX_CHOICES:
            raise ValueError(f"n must be between 1 and {MAX_CHOICES}")
        if self.logprobs is not None and not 0 <= int(self.logprobs) <= MAX_TOP_LOGPROBS:
            raise ValueError(f"logprobs must be between 0 and {MAX_TOP_LOGPROBS} alternatives")
        object.__setattr__(self, "stop_token_ids", tuple(int(t) for t in self.stop_token_ids))
        bias = tuple((int(t), float(b)) for t, b in self.logit_bias)
        if any(t < 0 for t, _ in bias) or len({t for t, _ in bias}) != len(bias):
            raise ValueError("logit_bias needs nonnegative token ids, each once")
        object.__setattr__(self, "logit_bias", bias)
        allowed = tuple(sorted({int(t) for t in self.allowed_token_ids}))
        if any(t < 0 for t in allowed):
            raise ValueError("allowed_token_ids must be nonnegative")
        object.__setattr__(self, "allowed_token_ids", allowed)
        words = tuple(tuple(int(t) for t in word) for word in self.bad_word_ids)
        if any(not word or any(t < 0 for t in word) for word in words):
            raise ValueError("bad_word_ids needs sequences of at least one nonnegative token id")
        object.__setattr__(self, "bad_word_ids", words)
        if self.timeout_secs is not None and not self.timeout_secs > 0.0:
            raise ValueError("timeout_secs must be positive")

    @property
    def penalizes(self) -> bool:
        """Whether tokens seen before change the logits (sampling.rs:98-107: what keeps a request off the plain argmax)."""
        return abs(self.repetition_penalty - 1.0) >= 1e-5 or self.presence_penalty != 0.0 or self.frequency_penalty != 0.0

    def adjusts_logits(self, generated: int) -> bool:
        """Whether the logits of the next token are changed before a token is chosen: penalties, biases, or
        end and stop ids that `min_tokens` still blocks after `generated` tokens."""
        return (self.penalizes or bool(self.logit_bias) or generated < self.min_tokens or bool(self.allowed_token_ids)
                or bool(self.bad_word_ids))

    @property
    def greedy(self) -> bool:
        return self.temperature <= GREEDY_TEMPERATURE

    def stops_on(self, token: int, eos: Sequence[int]) -> bool:
        """Explicit stop ids always stop; end-of-sequence ids unless ignored (sampling.rs:89-93)."""
        return token in self.stop_token_ids or (not self.ignore_eos and token in eos)

    def for_choice(self, index: int) -> "SamplingParams":
        """The parameters of the index-th answer: the same, with a seed of its own where one was given
        (rust/engine/src/runtime.rs:441-444); without a seed every sequence derives its own anyway."""
        if index == 0 or self.seed is None:
            return self
        from dataclasses import replace
        return replace(self, seed=(int(self.seed) + index * _CHOICE_SEED_STEP) & _MASK64)

    def seed_for(self, sequence_id: int) -> int:
        """sampling.rs:193-199: the request's seed, else one derived from the sequence id."""
        if self.seed is not None:
            return int(self.seed) & _MASK64
        return (_SEED_BASE ^ ((sequence_id * _SEED_STEP) & _MASK64)) & _MASK64
