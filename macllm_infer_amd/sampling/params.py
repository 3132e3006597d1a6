"""Sampling options, with the reference's names, meanings and defaults
(src/sampling.rs:14-33 ``SamplingConfig``; command-line flags src/main.rs:163-178)."""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Callable, Optional, Sequence, Tuple, Union


@dataclass(frozen=True)
class SamplingParams:
    max_new_tokens: int = 128
    temperature: float = 0.7          # 0 = greedy argmax
    top_k: int = 20                   # 0 (or >= vocabulary) = off
    top_p: float = 0.8                # 1.0 = off
    repetition_penalty: float = 1.1   # 1.0 = off; over prompt and generated tokens
    presence_penalty: float = 0.0     # over generated tokens only
    frequency_penalty: float = 0.0
    seed: int = 42
    ignore_eos: bool = False          # fixed-length runs (the reference's bench mode, src/main.rs:1169)
    stop_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    # A constraint on what may be generated (the reference masks the penalized logits through a constraint object,
    # src/sampling.rs:119-130): the token ids that may come next, every other logit counting as -inf; either a
    # fixed list, or a function of the tokens generated so far that returns the list for the next one (None: any
    # token).  A request with such a function has its tokens read before its next one is drawn.
    allowed_token_ids: Optional[Union[Tuple[int, ...], Callable[[Sequence[int]], Optional[Sequence[int]]]]] = None

    def __post_init__(self):
        # the reference's checks: src/sampling.rs:43-55, :67-75
        if not (math.isfinite(self.temperature) and self.temperature >= 0.0):
            raise ValueError("temperature must be finite and non-negative")
        if not (math.isfinite(self.top_p) and 0.0 < self.top_p <= 1.0):
            raise ValueError("top_p must be finite and in (0, 1]")
        if not (math.isfinite(self.repetition_penalty) and self.repetition_penalty > 0.0):
            raise ValueError("repetition_penalty must be finite and positive")
        if not (math.isfinite(self.presence_penalty) and -2.0 <= self.presence_penalty <= 2.0):
            raise ValueError("invalid presence_penalty")
        if not (math.isfinite(self.frequency_penalty) and -2.0 <= self.frequency_penalty <= 2.0):
            raise ValueError("invalid frequency_penalty")
        if self.top_k < 0:
            raise ValueError("top_k must be non-negative")
        if self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        object.__setattr__(self, "stop_token_ids", tuple(int(token) for token in self.stop_token_ids))
        if self.allowed_token_ids is not None and not callable(self.allowed_token_ids):
            allowed = tuple(int(token) for token in self.allowed_token_ids)
            if not allowed or min(allowed) < 0:
                raise ValueError("allowed_token_ids must name at least one token, none of them negative")
            object.__setattr__(self, "allowed_token_ids", allowed)

    @property
    def constrained_by_history(self) -> bool:
        return callable(self.allowed_token_ids)

    def allowed_after(self, generated: Sequence[int]) -> Optional[Tuple[int, ...]]:
        """The tokens that may follow ``generated``, or None for any."""
        if not callable(self.allowed_token_ids):
            return self.allowed_token_ids
        allowed = self.allowed_token_ids(generated)
        if allowed is None:
            return None
        allowed = tuple(int(token) for token in allowed)
        if not allowed or min(allowed) < 0:
            raise ValueError("the constraint rejected every token")           # src/sampling.rs:131-134
        return allowed

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    @property
    def uses_penalties(self) -> bool:
        return (abs(self.repetition_penalty - 1.0) >= 1.1920929e-07 or self.presence_penalty != 0.0
                or self.frequency_penalty != 0.0)


GREEDY = SamplingParams(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
