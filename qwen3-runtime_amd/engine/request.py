"""One request: its tokens, its options, what it has produced and why it stopped.

The engine speaks token ids. How many of the tokens are already in the cache is
the cache manager's knowledge, not the request's
(reference: qwen3_runtime/engine/request.py:29-131 keeps both on the request).
"""

from __future__ import annotations

import random
from enum import Enum, auto
from itertools import count
from typing import Sequence

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class Request:
    _ids = count()

    def __init__(
        self,
        token_ids: Sequence[int],
        max_tokens: int = 16,
        ignore_eos: bool = True,
        *,
        sampling: SamplingParams | None = None,
        stop_token_ids: Sequence[int] = (),
        forced_tokens: Sequence[int] | None = None,
        min_tokens: int | None = None,
    ):
        if not len(token_ids):
            raise ValueError("prompt token_ids must be non-empty")
        if max_tokens < 1:
            raise ValueError("max_tokens must be positive")
        self.request_id = next(Request._ids)
        self.status = RequestStatus.WAITING
        self.token_ids = [int(t) for t in token_ids]
        self.num_prompt_tokens = len(self.token_ids)
        self.max_tokens = int(max_tokens)
        self.ignore_eos = bool(ignore_eos)
        self.sampling = sampling or SamplingParams()
        self.stop_token_ids = tuple(int(t) for t in stop_token_ids)
        self.min_tokens = int(self.sampling.min_tokens if min_tokens is None else min_tokens)
        self.forced_tokens = None if forced_tokens is None else [int(t) for t in forced_tokens]
        # no seed: one is drawn now, so that the request is still reproducible from its record
        # (reference: qwen3_runtime/sampling.py:293-298 falls back to the global generator)
        self.seed = self.sampling.seed if self.sampling.seed is not None else random.getrandbits(62)
        self.num_scheduled_tokens = 0
        self.num_preemptions = 0
        self.admitted = False  # holds a state slot
        self.logprobs: list[float] = []
        self.finish_reason: str | None = None

    def __len__(self) -> int:
        return len(self.token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def output_tokens(self) -> list[int]:
        return self.token_ids[self.num_prompt_tokens:]

    def next_forced_token(self) -> int | None:
        """Next teacher-forced id, if any (reference: qwen3_runtime/engine/request.py:101-108)."""
        if self.forced_tokens is None:
            return None
        produced = self.num_output_tokens
        return self.forced_tokens[produced] if produced < len(self.forced_tokens) else None
