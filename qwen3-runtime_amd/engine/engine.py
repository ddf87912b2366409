"""The engine loop: decide a step, run it, sample, settle.

``add_request`` queues a request and returns its id. ``step()`` asks the
scheduler who takes part, hands their next tokens to the step function, samples
for every request whose tokens are now all in the cache, and reports
``[(request id, new token or None, ended)]`` (reference, for the same contract:
qwen3_runtime/engine/engine.py:53-92,216-260). ``generate`` and
``generate_batch`` drive ``step()`` until their requests have ended.
"""

from __future__ import annotations

import math
from typing import Iterator, Sequence

from ..config.engine import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request
from .scheduler import Scheduler


class Engine:
    def __init__(self, config: EngineConfig, loaded):
        self.config = config
        self.loaded = loaded
        self.cache = loaded.cache
        self.runner = loaded.runner
        self.scheduler = Scheduler(config, self.cache, self.runner.max_model_len,
                                   portion_multiple=loaded.model.portion_multiple)
        self.sampler = Sampler(self.runner.ops, self.cache.slots, self.runner.vocab_size, self.runner.device)
        self._live: dict[int, Request] = {}
        self.last_step_stats: dict | None = None
        self._broken: str | None = None

    # ---- requests ----------------------------------------------------------------
    def add_request(self, token_ids: Sequence[int], max_tokens: int = 16, *, ignore_eos: bool = True,
                    sampling: SamplingParams | None = None, stop_token_ids: Sequence[int] = (),
                    forced_tokens: Sequence[int] | None = None) -> int:
        self._refuse_if_broken()
        req = Request(token_ids, max_tokens, ignore_eos, sampling=sampling, stop_token_ids=stop_token_ids,
                      forced_tokens=forced_tokens)
        self._check_ids(req)
        self.scheduler.add(req)
        self._live[req.request_id] = req
        return req.request_id

    def _check_ids(self, req: Request) -> None:
        """Every id that will index device memory (the embedding table, a row of logits, the
        penalty counts) is checked here, on the host: a kernel cannot report a bad index, it
        can only write where it must not."""
        vocab = self.runner.vocab_size
        bias = req.sampling.logit_bias or {}
        for what, ids in (("prompt token", req.token_ids), ("forced token", req.forced or ()),
                          ("logit_bias key", list(bias))):
            for t in ids:
                if isinstance(t, bool) or int(t) != t or not 0 <= int(t) < vocab:
                    raise ValueError(f"{what} {t!r} is outside the vocabulary of {vocab} ids")
        for t, v in bias.items():
            v = float(v)
            if math.isnan(v) or v == math.inf:
                raise ValueError(f"logit_bias[{t}] = {v}: a bias is a finite number, or -inf to exclude the id")

    def request(self, request_id: int) -> Request:
        return self._live[request_id]

    def finish_request(self, request_id: int) -> None:
        """Cancel: the request ends now and gives back what it holds."""
        req = self._live.pop(request_id, None)
        if req is not None:
            self.scheduler.retire(req, "abort")

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ---- one step -------------------------------------------------------------------
    def _refuse_if_broken(self) -> None:
        """A step that failed on the device side leaves the cache's books and the device's
        contents in disagreement; nothing more is run on them
        (reference: qwen3_runtime/engine/engine.py:210-225)."""
        if self._broken is not None:
            raise RuntimeError("engine terminated after a failed step: " + self._broken)

    def step(self) -> list[tuple[int, int | None, bool]]:
        self._refuse_if_broken()
        evictions = self.scheduler.num_preemptions
        batch = self.scheduler.schedule()
        if not batch:
            self.last_step_stats = None
            if not self.scheduler.is_finished():
                raise RuntimeError("scheduler produced an empty step while requests remain")
            return []
        try:
            return self._run_step(batch, evictions)
        except BaseException as exc:
            self._broken = f"{type(exc).__name__}: {exc}"
            raise

    def _next_step_is_known(self, batch: list[Request], to_sample: list[Request]) -> bool:
        """Whatever ids this step's sampling gives, the next step is the same requests with one
        token each: all of them decode, none can end with the next token (stop ids do not count
        for it and its limit is further off), and nobody else holds pages or waits."""
        if len(to_sample) != len(batch) or self.scheduler.queue or len(self.scheduler.residents) != len(batch):
            return False
        return all(r.grant == 1 and not r.stop.stop_ids_count and r.num_output_tokens + 1 < r.stop.limit
                   for r in batch)

    def _run_step(self, batch: list[Request], evictions_before: int):
        entries, to_sample, spans = [], [], []
        n_prompt = n_decode = 0
        for req in batch:
            at = self.cache.length(req.request_id)
            if at == 0 and req.restarts == 0:  # its first step: options and seed go into its slot
                self.sampler.admit(self.cache.slots.slot(req.request_id), req.sampling, req.seed,
                                   req.token_ids[: req.prompt_len])
            upto = at + req.grant
            caught_up = upto >= len(req.token_ids)
            spans.append((req.grant, upto))
            entries.append(StepEntry(req.request_id, req.token_ids[at:upto], [req.grant - 1] if caught_up else []))
            if caught_up:
                to_sample.append(req)
            if at >= req.prompt_len:
                n_decode += req.grant
            else:
                n_prompt += req.grant
        logits = self.runner.step(entries)
        new_token: dict[int, int] = {}
        if to_sample:
            # the rows' state slots went to the device with the step's other arrays
            slot_rows = self.runner.last_row_slots
            if logits is None or slot_rows is None or slot_rows.numel() != len(to_sample):
                raise RuntimeError("the step's logits do not match the requests to sample for")
            drawn = self.sampler.launch(logits, slot_rows, to_sample)
            if self._next_step_is_known(batch, to_sample):
                # the device goes on with the next step while the host waits for this one's ids
                self.runner.step_ahead(drawn.tokens)
            ids, logprobs = self.sampler.finish(drawn)
            for req, tok, lp in zip(to_sample, ids, logprobs):
                new_token[req.request_id] = tok
                req.logprobs.append(lp)
        sampled = [new_token.get(req.request_id) for req in batch]
        ended = {req.request_id for req in self.scheduler.settle(batch, sampled)}
        for rid in ended:
            self._live.pop(rid, None)
        self.last_step_stats = {
            "req_ids": [req.request_id for req in batch],
            "spans": spans,  # per request: (tokens of the step, tokens in the cache after it)
            "prefill_tokens": n_prompt,
            "decode_tokens": n_decode,
            "preempts": self.scheduler.num_preemptions - evictions_before,
        }
        return [(req.request_id, tok, req.request_id in ended) for req, tok in zip(batch, sampled)]

    # ---- whole requests ------------------------------------------------------------------
    def _drive(self, reqs: Sequence[Request]) -> Iterator[list[tuple[int, int | None, bool]]]:
        while not all(r.done for r in reqs):
            results = self.step()
            if not results:
                raise RuntimeError("no progress while requests remain")
            yield results

    def stream_request(self, request_id: int) -> Iterator[int]:
        """The request's new tokens as they come (other queued requests advance as well)."""
        for results in self._drive([self._live[request_id]]):
            for rid, tok, _ended in results:
                if rid == request_id and tok is not None:
                    yield tok

    def generate(self, token_ids: Sequence[int], max_tokens: int = 16, **options) -> list[int]:
        return list(self.stream_request(self.add_request(token_ids, max_tokens=max_tokens, **options)))

    def generate_batch(self, prompts: Sequence[Sequence[int]], max_tokens: int = 16, sampling=None,
                       **options) -> list[list[int]]:
        """All prompts are queued at once and batched continuously; outputs in the order given."""
        per_prompt = sampling if isinstance(sampling, (list, tuple)) else [sampling] * len(prompts)
        reqs = [self._live[self.add_request(p, max_tokens=max_tokens, sampling=s, **options)]
                for p, s in zip(prompts, per_prompt)]
        for _ in self._drive(reqs):
            pass
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
