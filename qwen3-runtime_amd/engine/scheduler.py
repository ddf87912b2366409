"""Continuous batching with prompts cut into portions under a token budget.

One ``schedule()`` call decides a step: running requests first, in admission
order (a decoding request takes one token, an unfinished prompt a portion),
then waiting requests while the token budget and ``max_num_seqs`` allow. A
portion is ``min(uncomputed, budget)``, shrunk to what the request's held pages
plus the free pages can store. Pages are reserved only for the step's tokens
(reference: qwen3_runtime/engine/scheduler.py:47-64,227-295).

When pages run out: a running request that cannot get a page sits the step
out. If no request at all can be scheduled, the youngest running request is
preempted: its pages go back, it keeps its tokens (prompt and output), its
state slot and its place at the front of the waiting queue, and is computed
again from position 0 later; it samples again only when it has caught up
(reference: qwen3_runtime/engine/scheduler.py:56-58,297-306). If nothing is
running and the first waiting request still cannot get a page, that is an
error. A request whose prompt plus ``max_tokens`` can never fit the pool or the
position limit is refused when it is added
(reference: qwen3_runtime/engine/scheduler.py:34-42).
"""

from __future__ import annotations

from collections import deque

from ..cache import CacheManager
from ..config.engine import EngineConfig
from .request import Request, RequestStatus


class Scheduler:
    def __init__(self, config: EngineConfig, cache: CacheManager, max_model_len: int):
        self.config = config
        self.cache = cache
        self.max_model_len = int(max_model_len)
        self.waiting: deque[Request] = deque()
        self.running: deque[Request] = deque()
        self.num_preemptions = 0

    # ---- queue ---------------------------------------------------------------
    def add(self, req: Request) -> None:
        max_len = len(req.token_ids) + req.max_tokens
        # the last sampled token is never fed back, so it needs neither a page nor a position
        if max_len - 1 > self.max_model_len:
            raise RuntimeError(
                f"request length {max_len} exceeds the model's limit of {self.max_model_len} positions"
            )
        needed = self.cache.pages_needed_for(max_len)
        if self.cache.groups and needed > self.cache.num_pages:
            raise RuntimeError(
                f"request length {max_len} needs {needed} cache pages; the pool has {self.cache.num_pages}"
            )
        req.status = RequestStatus.WAITING
        self.waiting.append(req)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def computed(self, req: Request) -> int:
        return self.cache.length(req.request_id) if req.admitted else 0

    def uncomputed(self, req: Request) -> int:
        return max(0, len(req.token_ids) - self.computed(req))

    # ---- one step's decision ---------------------------------------------------
    def schedule(self) -> list[Request]:
        bound = self.config.max_num_seqs + len(self.running) + len(self.waiting) + 1
        for _ in range(bound):
            scheduled: list[Request] = []
            budget = self._schedule_running(scheduled, self.config.max_num_batched_tokens)
            self._schedule_waiting(scheduled, budget)
            if scheduled:
                return scheduled
            if self.running:
                self._preempt(self.running.pop())
                continue
            if self.waiting:
                raise RuntimeError("the first waiting request cannot get a cache page although nothing is running")
            return []
        raise RuntimeError("scheduler could not form a step after preempting every request")

    def _portion(self, req: Request, budget: int) -> int:
        remaining = self.uncomputed(req)
        if remaining <= 0 or budget <= 0:
            return 0
        return self.cache.max_reservable_tokens(req.request_id, min(remaining, budget))

    def _schedule_running(self, scheduled: list[Request], budget: int) -> int:
        for req in self.running:
            if len(scheduled) >= self.config.max_num_seqs or budget <= 0:
                break
            n = self._portion(req, budget)
            if n <= 0:
                continue  # no page for it now: it sits this step out
            self.cache.reserve(req.request_id, n)
            req.num_scheduled_tokens = n
            scheduled.append(req)
            budget -= n
        return budget

    def _schedule_waiting(self, scheduled: list[Request], budget: int) -> None:
        deferred: list[Request] = []
        while self.waiting:
            if len(scheduled) >= self.config.max_num_seqs or budget <= 0:
                break
            req = self.waiting.popleft()
            if not req.admitted:
                if self.cache.slots.num_free == 0:
                    deferred.append(req)
                    break  # later requests must not overtake it for a slot
                self.cache.admit(req.request_id)
                req.admitted = True
            n = self._portion(req, budget)
            if n <= 0:
                deferred.append(req)
                continue
            self.cache.reserve(req.request_id, n)
            req.num_scheduled_tokens = n
            req.status = RequestStatus.RUNNING
            scheduled.append(req)
            self.running.append(req)
            budget -= n
        self.waiting.extendleft(reversed(deferred))

    def _preempt(self, req: Request) -> None:
        self.cache.restart(req.request_id)
        req.num_scheduled_tokens = 0
        req.num_preemptions += 1
        req.status = RequestStatus.WAITING
        self.waiting.appendleft(req)
        self.num_preemptions += 1

    # ---- after the step ----------------------------------------------------------
    def postprocess(self, reqs: list[Request], token_ids: list[int | None]) -> list[Request]:
        """The step's tokens are in the cache; append sampled tokens; finish what is done
        (reference: qwen3_runtime/engine/scheduler.py:66-87)."""
        if len(token_ids) != len(reqs):
            raise ValueError("token_ids must align with scheduled requests")
        finished = []
        for req, tok in zip(reqs, token_ids):
            req.num_scheduled_tokens = 0
            if tok is None:
                continue
            req.token_ids.append(int(tok))
            reason = self._finish_reason(req)
            if reason is not None:
                req.finish_reason = reason
                self.finish(req)
                finished.append(req)
        return finished

    def _finish_reason(self, req: Request) -> str | None:
        """Stop ids count only when ``ignore_eos`` is off and ``min_tokens`` are out; then length
        (reference: qwen3_runtime/engine/scheduler.py:106-122)."""
        n_out = req.num_output_tokens
        tok = req.token_ids[-1]
        hit_stop = (not req.ignore_eos) and (
            tok in req.stop_token_ids
            or (self.config.eos_token_id is not None and tok == self.config.eos_token_id)
        )
        if hit_stop and n_out >= req.min_tokens:
            return "stop"
        if n_out >= req.max_tokens:
            return "length"
        return None

    def finish(self, req: Request) -> None:
        """Give back pages and slot; also the way to cancel a request."""
        req.status = RequestStatus.FINISHED
        if req.admitted:
            self.cache.release(req.request_id)
            req.admitted = False
        for queue in (self.running, self.waiting):
            try:
                queue.remove(req)
            except ValueError:
                pass
