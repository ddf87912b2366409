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
        def finite(name: str) -> float:
            value = float(getattr(self, name))
            if not math.isfinite(value):
                raise ValueError(f"{name} is {value}; it has to be a finite number")
            return value

        finite("temperature")
        if not 0.0 < finite("top_p") <= 1.0:
            raise ValueError(f"top_p is {self.top_p}; it is a probability mass in (0, 1]")
        if not 0.0 <= finite("min_p") <= 1.0:
            raise ValueError(f"min_p is {self.min_p}; it is a share of the largest probability, in [0, 1]")
        if finite("repetition_penalty") <= 0.0:
            raise ValueError(f"repetition_penalty is {self.repetition_penalty}; logits are divided by it, so it is > 0")
        finite("presence_penalty")
        finite("frequency_penalty")
        if self.min_tokens < 0:
            raise ValueError(f"min_tokens is {self.min_tokens}; a count of tokens cannot be negative")

    def is_greedy(self) -> bool:
        return self.temperature <= 0.0

    def has_penalties(self) -> bool:
        return (self.repetition_penalty, self.presence_penalty, self.frequency_penalty) != (1.0, 0.0, 0.0)
