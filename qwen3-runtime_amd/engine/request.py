"""One request as the engine sees it: token ids in, token ids out, and when to stop.

A request owns its tokens (prompt, then whatever was sampled), its sampling
options and a ``StopRule``. It does not know how many of its tokens are in the
cache: that is the cache manager's book, read through ``CacheManager.length``
(the reference keeps that count on the request, qwen3_runtime/engine/request.py:29-131).
"""

from __future__ import annotations

import enum
import itertools
import random
from dataclasses import dataclass
from typing import Sequence

from ..sampling.params import SamplingParams

_next_id = itertools.count()


class Phase(enum.Enum):
    QUEUED = "queued"      # waits for a step (new, or sent back to recompute)
    RUNNING = "running"    # took part in a step and holds pages
    DONE = "done"


@dataclass(frozen=True)
class StopRule:
    """When a request ends. Stop ids (the model's end-of-sequence id and the request's own)
    count only if ``stop_ids_count`` and only once ``floor`` tokens are out; the length limit
    always counts, after them (reference: qwen3_runtime/engine/scheduler.py:106-122)."""

    limit: int
    floor: int = 0
    stop_ids_count: bool = False
    stop_ids: frozenset = frozenset()

    def verdict(self, produced: int, last_token: int, eos_token_id: int | None) -> str | None:
        if self.stop_ids_count and produced >= self.floor:
            if last_token in self.stop_ids or (eos_token_id is not None and last_token == eos_token_id):
                return "stop"
        return "length" if produced >= self.limit else None


class Request:
    """``Request(prompt, max_tokens, ignore_eos, sampling=, stop_token_ids=, forced_tokens=,
    min_tokens=)``: the options of the reference's ``Engine.add_request``
    (qwen3_runtime/engine/engine.py:53-65) that this engine has."""

    def __init__(self, token_ids: Sequence[int], max_tokens: int = 16, ignore_eos: bool = True, *,
                 sampling: SamplingParams | None = None, stop_token_ids: Sequence[int] = (),
                 forced_tokens: Sequence[int] | None = None, min_tokens: int | None = None):
        prompt = [int(t) for t in token_ids]
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if int(max_tokens) < 1:
            raise ValueError(f"max_tokens is {max_tokens}; a request produces at least one token")
        self.request_id = next(_next_id)
        self.sampling = sampling if sampling is not None else SamplingParams()
        self.stop = StopRule(
            limit=int(max_tokens),
            floor=int(self.sampling.min_tokens if min_tokens is None else min_tokens),
            stop_ids_count=not ignore_eos,
            stop_ids=frozenset(int(t) for t in stop_token_ids),
        )
        self.token_ids = prompt            # grows by one per sampled token
        self.prompt_len = len(prompt)
        self.forced = None if forced_tokens is None else tuple(int(t) for t in forced_tokens)
        # A request without a seed gets one here, so that its record still reproduces it
        # (the reference falls back to the global generator: qwen3_runtime/sampling.py:293-298).
        self.seed = self.sampling.seed if self.sampling.seed is not None else random.getrandbits(62)
        self.logprobs: list[float] = []
        self.phase = Phase.QUEUED
        self.finish_reason: str | None = None
        # the scheduler's notes
        self.grant = 0            # tokens of this request in the step being run
        self.restarts = 0         # times it lost its pages and started over
        self.holds_slot = False   # has a state slot (from its first step to its end)

    # ---- what it has produced ----------------------------------------------------
    @property
    def max_tokens(self) -> int:
        return self.stop.limit

    @property
    def num_output_tokens(self) -> int:
        return len(self.token_ids) - self.prompt_len

    @property
    def output_tokens(self) -> list[int]:
        return self.token_ids[self.prompt_len:]

    @property
    def done(self) -> bool:
        return self.phase is Phase.DONE

    def accept(self, token: int, eos_token_id: int | None) -> str | None:
        """Append a sampled token; returns why the request ends with it, or None."""
        self.token_ids.append(int(token))
        return self.stop.verdict(self.num_output_tokens, self.token_ids[-1], eos_token_id)

    def forced_next(self) -> int | None:
        """With teacher forcing (reference: qwen3_runtime/engine/request.py:101-108): the id the
        next output position must take, while the given list lasts."""
        i = self.num_output_tokens
        return self.forced[i] if self.forced is not None and i < len(self.forced) else None

    def __repr__(self) -> str:
        return (f"Request({self.request_id}, {self.phase.value}, prompt {self.prompt_len}, "
                f"out {self.num_output_tokens}/{self.stop.limit})")
