"""Per-request sampling options.  Names, defaults and the ranges that are accepted are the reference's
(``engine/utils.py:9-47``): they are the schema callers write against."""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    n: int = 1
    temperature: float = 1.0
    top_p: float = 1.0
    top_k: int = 0
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    ignore_eos: bool = False
    max_tokens: int = 512
    seed: Optional[int] = None
    stop_token_ids: List[int] = field(default_factory=list)

    def __post_init__(self) -> None:
        problems = []
        if self.n != 1:
            problems.append(f"n={self.n}: one sequence is generated per request")
        if not self.temperature >= 0.0 or math.isinf(self.temperature):
            problems.append(f"temperature={self.temperature}: a finite number >= 0 (0 = greedy)")
        if not 0.0 < self.top_p <= 1.0:
            problems.append(f"top_p={self.top_p}: a share of the probability mass, above 0 and at most 1")
        if self.top_k < 0:
            problems.append(f"top_k={self.top_k}: a count of tokens to keep, 0 = no limit")
        if not self.repetition_penalty > 0.0:
            problems.append(f"repetition_penalty={self.repetition_penalty}: a factor above 0 (1 = none)")
        if self.max_tokens < 1:
            problems.append(f"max_tokens={self.max_tokens}: a request generates at least one token")
        if problems:
            raise ValueError("sampling options out of range: " + "; ".join(problems))

    @property
    def is_greedy(self) -> bool:
        return self.temperature == 0.0

    @property
    def has_penalties(self) -> bool:
        return (self.repetition_penalty, self.presence_penalty, self.frequency_penalty) != (1.0, 0.0, 0.0)
