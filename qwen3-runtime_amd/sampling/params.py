"""Sampling options of one request.

Names, defaults and validation follow the reference's ``SamplingParams``
(qwen3_runtime/sampling_params.py:9-46). The chain runs in the order the
reference executes it (qwen3_runtime/sampling.py:120-135): logit bias,
penalties, (greedy stops here), temperature, min_p, top_k, top_p, softmax, draw.
``temperature <= 0`` is greedy: the first maximal id.
"""

from __future__ import annotations

import math
from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = 0
    min_p: float = 0.0
    seed: int | None = None
    repetition_penalty: float = 1.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    logit_bias: dict[int, float] | None = None
    min_tokens: int = 0
    logprobs: bool = False

    def __post_init__(self) -> None:
        if not math.isfinite(self.temperature):
            raise ValueError("temperature must be finite")
        if not math.isfinite(self.top_p) or not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must satisfy 0 < top_p <= 1")
        if not math.isfinite(self.min_p) or not 0.0 <= self.min_p <= 1.0:
            raise ValueError("min_p must satisfy 0 <= min_p <= 1")
        if self.min_tokens < 0:
            raise ValueError("min_tokens must be non-negative")
        if self.repetition_penalty <= 0 or not math.isfinite(self.repetition_penalty):
            raise ValueError("repetition_penalty must be positive and finite")
        for name in ("presence_penalty", "frequency_penalty"):
            if not math.isfinite(getattr(self, name)):
                raise ValueError(f"{name} must be finite")

    def is_greedy(self) -> bool:
        return self.temperature <= 0.0

    def has_penalties(self) -> bool:
        return not (
            self.repetition_penalty == 1.0
            and self.presence_penalty == 0.0
            and self.frequency_penalty == 0.0
        )
