"""Who takes part in the next step, and with how many tokens.

A step has two limits: ``max_num_batched_tokens`` tokens and ``max_num_seqs``
requests. Candidates are walked in one fixed order, residents (requests that
hold pages, oldest first) and then the queue (arrival order), and each is
offered ``min(what it still has to compute, what is left of the token limit)``,
cut down to the tokens its own pages plus the free pages can hold. A decoding
request therefore takes one token and a prompt is cut into portions; pages are
taken for the step's tokens only. These are the reference's rules
(qwen3_runtime/engine/scheduler.py:47-64,227-295); the walk over one candidate
list is this file's own.

When pages run out. A candidate whose offer comes to nothing is passed over for
this step: a resident waits with its pages, a queued request keeps its place.
If the whole walk yields nothing, the newest resident is sent back to the head
of the queue: its pages return to the pool, it keeps its tokens (prompt and
output so far) and its state slot, and will be computed again from position 0,
sampling again only when it has caught up
(reference: qwen3_runtime/engine/scheduler.py:56-58,297-306). With no resident
left and the head of the queue still without a page the pool is held by
someone else: an error. A request whose prompt plus ``max_tokens`` can never
fit the pool or the position limit is refused on arrival
(reference: qwen3_runtime/engine/scheduler.py:34-42).
"""

from __future__ import annotations

from collections import deque

from ..cache import CacheManager
from ..config.engine import EngineConfig
from .request import Phase, Request


class Scheduler:
    def __init__(self, config: EngineConfig, cache: CacheManager, max_model_len: int,
                 portion_multiple: int = 1):
        self.config = config
        self.cache = cache
        self.max_model_len = int(max_model_len)
        # a portion that does not end its request's tokens is a multiple of this many tokens
        # (a mixer that works in blocks of its own asks for it; 1 for attention)
        self.portion_multiple = max(1, int(portion_multiple))
        self.queue: deque[Request] = deque()
        self.residents: list[Request] = []
        self.num_preemptions = 0

    # ---- arrivals ------------------------------------------------------------------
    def add(self, req: Request) -> None:
        longest = len(req.token_ids) + req.max_tokens
        # the last sampled token is never fed back, so it needs neither a page nor a position
        if longest - 1 > self.max_model_len:
            raise RuntimeError(
                f"request length {longest} exceeds the model's limit of {self.max_model_len} positions")
        # per group of caches: one that keeps a window of keys needs the window's pages only
        fits, why_not = self.cache.can_ever_hold(longest)
        if not fits:
            raise RuntimeError(why_not)
        req.phase = Phase.QUEUED
        self.queue.append(req)

    def is_finished(self) -> bool:
        return not self.queue and not self.residents

    def behind(self, req: Request) -> int:
        """Tokens of the request that are not in the cache yet."""
        stored = self.cache.length(req.request_id) if req.holds_slot else 0
        return len(req.token_ids) - stored

    # ---- one step's decision ---------------------------------------------------------
    def schedule(self) -> list[Request]:
        # Pages that a replayed decode step took ahead for its requests' next tokens go back to the
        # pool before anybody is offered anything, whenever somebody besides a decoding resident
        # wants pages (residents are walked first and take theirs again): what a candidate is
        # offered then never depends on what the step function did ahead of the books.
        if self.queue or any(self.behind(r) > 1 for r in self.residents):
            self.cache.trim()
        while True:
            step = self._walk()
            if step:
                return step
            if not self.residents:
                if self.queue:
                    raise RuntimeError(
                        "the first waiting request cannot get a cache page although nothing is running")
                return []
            self._send_back(self.residents[-1])  # at most once per resident: the loop ends

    def _offer(self, req: Request, tokens_left: int) -> int:
        want = min(self.behind(req), tokens_left)
        if want <= 0:
            return 0
        n = self.cache.max_reservable_tokens(req.request_id, want)
        if n < self.behind(req) and self.portion_multiple > 1:
            n -= n % self.portion_multiple
        return max(0, n)

    def _walk(self) -> list[Request]:
        tokens_left, seats_left = self.config.max_num_batched_tokens, self.config.max_num_seqs
        step: list[Request] = []
        for req in self.residents + list(self.queue):
            if tokens_left <= 0 or seats_left <= 0:
                break
            if not req.holds_slot:
                if self.cache.slots.num_free == 0:
                    break  # nobody behind it in the queue may take the next free slot
                self.cache.admit(req.request_id)
                req.holds_slot = True
            n = self._offer(req, tokens_left)
            if n == 0:
                continue
            self.cache.reserve(req.request_id, n)
            req.grant = n
            tokens_left -= n
            seats_left -= 1
            step.append(req)
        for req in step:
            if req.phase is Phase.QUEUED:
                self.queue.remove(req)
                self.residents.append(req)
                req.phase = Phase.RUNNING
        return step

    def _send_back(self, req: Request) -> None:
        self.cache.restart(req.request_id)
        self.residents.remove(req)
        self.queue.appendleft(req)
        req.phase, req.grant = Phase.QUEUED, 0
        req.restarts += 1
        self.num_preemptions += 1

    # ---- after the step ------------------------------------------------------------------
    def settle(self, step: list[Request], sampled: list[int | None]) -> list[Request]:
        """The step's tokens are in the cache. ``sampled[i]`` is the new token of ``step[i]``, or
        None for a portion that did not reach the end of its request's tokens. Returns the
        requests that ended (reference: qwen3_runtime/engine/scheduler.py:66-87)."""
        if len(sampled) != len(step):
            raise ValueError(f"{len(sampled)} sampled tokens for a step of {len(step)} requests")
        ended = []
        for req, token in zip(step, sampled):
            req.grant = 0
            if token is None:
                continue
            reason = req.accept(token, self.config.eos_token_id)
            if reason is not None:
                self.retire(req, reason)
                ended.append(req)
        return ended

    def retire(self, req: Request, reason: str) -> None:
        """The request ends (also: is cancelled): pages and slot go back."""
        if req.done:
            return
        if req in self.residents:
            self.residents.remove(req)
        elif req in self.queue:
            self.queue.remove(req)
        if req.holds_slot:
            self.cache.release(req.request_id)
            req.holds_slot = False
        req.phase, req.finish_reason = Phase.DONE, req.finish_reason or reason
