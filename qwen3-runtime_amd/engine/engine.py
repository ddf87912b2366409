"""The engine loop: schedule, run one step, sample, finish.

``add_request`` queues a request; ``step()`` asks the scheduler for a batch,
runs it through the step function, samples the rows that reached the end of
their tokens and returns ``[(request id, new token or None, finished)]``
(reference: qwen3_runtime/engine/engine.py:53-92,216-260).
"""

from __future__ import annotations

from typing import Iterator, Sequence

import torch

from ..config.engine import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request, RequestStatus
from .scheduler import Scheduler


class Engine:
    def __init__(self, config: EngineConfig, loaded):
        self.config = config
        self.loaded = loaded
        self.cache = loaded.cache
        self.runner = loaded.runner
        self.scheduler = Scheduler(config, self.cache, self.runner.max_model_len)
        self.sampler = Sampler(self.runner.ops, self.cache.slots, self.runner.vocab_size, self.runner.device)
        self._requests: dict[int, Request] = {}
        self.last_step_stats: dict | None = None
        self._fatal_error: str | None = None

    # ---- requests --------------------------------------------------------------
    def add_request(
        self,
        token_ids: Sequence[int],
        max_tokens: int = 16,
        *,
        ignore_eos: bool = True,
        sampling: SamplingParams | None = None,
        stop_token_ids: Sequence[int] = (),
        forced_tokens: Sequence[int] | None = None,
    ) -> int:
        self._check_health()
        req = Request(token_ids, max_tokens, ignore_eos, sampling=sampling,
                      stop_token_ids=stop_token_ids, forced_tokens=forced_tokens)
        bad = [t for t in req.token_ids if not 0 <= t < self.runner.vocab_size]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary of {self.runner.vocab_size}")
        self.scheduler.add(req)
        self._requests[req.request_id] = req
        return req.request_id

    def request(self, request_id: int) -> Request:
        return self._requests[request_id]

    def finish_request(self, request_id: int) -> None:
        """Cancel: give back what the request holds."""
        req = self._requests.pop(request_id, None)
        if req is not None and req.status != RequestStatus.FINISHED:
            req.finish_reason = req.finish_reason or "abort"
            self.scheduler.finish(req)

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ---- one step -----------------------------------------------------------------
    def _check_health(self) -> None:
        """After a failure on the device side of a step the cache's books and the device's state
        no longer agree: the engine refuses further work
        (reference: qwen3_runtime/engine/engine.py:210-225)."""
        if self._fatal_error is not None:
            raise RuntimeError("engine terminated after a failed step: " + self._fatal_error)

    def step(self) -> list[tuple[int, int | None, bool]]:
        self._check_health()
        preempt_before = self.scheduler.num_preemptions
        reqs = self.scheduler.schedule()
        if not reqs:
            self.last_step_stats = None
            if not self.scheduler.is_finished():
                raise RuntimeError("scheduler produced an empty step while requests remain")
            return []
        entries, sampling_reqs = [], []
        prefill_tokens = decode_tokens = 0
        for req in reqs:
            start = self.cache.length(req.request_id)
            n = req.num_scheduled_tokens
            if start == 0 and req.num_preemptions == 0:
                self.sampler.admit(self.cache.slots.slot(req.request_id), req.sampling, req.seed,
                                   req.token_ids[: req.num_prompt_tokens])
            reaches_end = start + n >= len(req.token_ids)
            entries.append(StepEntry(req.request_id, req.token_ids[start: start + n],
                                     [n - 1] if reaches_end else []))
            if reaches_end:
                sampling_reqs.append(req)
            if start >= req.num_prompt_tokens:
                decode_tokens += n
            else:
                prefill_tokens += n
        try:
            return self._run(reqs, entries, sampling_reqs, prefill_tokens, decode_tokens, preempt_before)
        except BaseException as exc:
            self._fatal_error = f"{type(exc).__name__}: {exc}"
            raise

    def _run(self, reqs, entries, sampling_reqs, prefill_tokens, decode_tokens, preempt_before):
        logits = self.runner.step(entries)
        tokens: list[int | None] = [None] * len(reqs)
        if sampling_reqs:
            # the rows' state slots went up with the step's other arrays: no copy, no wait here
            slot_rows = self.runner.last_row_slots
            if slot_rows is None or slot_rows.numel() != len(sampling_reqs):
                raise RuntimeError("the step's logits do not match the requests to sample for")
            sampled, logprobs = self.sampler.sample(logits, slot_rows, sampling_reqs)
            by_id = {r.request_id: (t, lp) for r, t, lp in zip(sampling_reqs, sampled, logprobs)}
            for i, req in enumerate(reqs):
                if req.request_id in by_id:
                    tokens[i], lp = by_id[req.request_id]
                    req.logprobs.append(lp)
        finished = {r.request_id for r in self.scheduler.postprocess(reqs, tokens)}
        self.last_step_stats = {
            "req_ids": [r.request_id for r in reqs],
            "prefill_tokens": prefill_tokens,
            "decode_tokens": decode_tokens,
            "preempts": self.scheduler.num_preemptions - preempt_before,
        }
        for rid in finished:
            self._requests.pop(rid, None)
        return [(r.request_id, t, r.request_id in finished) for r, t in zip(reqs, tokens)]

    # ---- whole requests --------------------------------------------------------------
    def stream_request(self, request_id: int) -> Iterator[int]:
        """Yield the request's new tokens until it finishes (other requests advance too)."""
        req = self._requests[request_id]
        while req.status != RequestStatus.FINISHED:
            progressed = False
            for rid, tok, _done in self.step():
                progressed = True
                if rid == request_id and tok is not None:
                    yield tok
            if not progressed:
                raise RuntimeError(f"request {request_id} made no progress")

    def generate(self, token_ids: Sequence[int], max_tokens: int = 16, **kwargs) -> list[int]:
        return list(self.stream_request(self.add_request(token_ids, max_tokens=max_tokens, **kwargs)))

    def generate_batch(self, prompts: Sequence[Sequence[int]], max_tokens: int = 16, sampling=None,
                       **kwargs) -> list[list[int]]:
        """All prompts are queued at once and batched continuously; outputs in the order given."""
        samplings = sampling if isinstance(sampling, (list, tuple)) else [sampling] * len(prompts)
        reqs = []
        for p, s in zip(prompts, samplings):
            rid = self.add_request(p, max_tokens=max_tokens, sampling=s, **kwargs)
            reqs.append(self._requests[rid])
        while any(r.status != RequestStatus.FINISHED for r in reqs):
            if not self.step():
                raise RuntimeError("no progress while requests remain")
        return [r.output_tokens for r in reqs]

    def config_report(self) -> dict:
        """The settings in effect (reference: qwen3_runtime/engine/engine.py:150-181)."""
        return {
            "page_size": self.config.page_size,
            "num_pages": self.cache.num_pages,
            "max_num_seqs": self.config.max_num_seqs,
            "max_num_batched_tokens": self.config.max_num_batched_tokens,
            "dtype": self.config.dtype,
            "hip_graph": self.runner.hip_graph,
            "max_model_len": self.runner.max_model_len,
            "weight_bytes": self.loaded.weight_bytes,
        }
