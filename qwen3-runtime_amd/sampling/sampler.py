"""Sampling of a step's rows on the device, with per-request state in slots.

A request's options, its seed and the index of its next draw are written into
its state slot when it is admitted; penalty counts (occurrences of every id in
prompt and output) sit in the same slot. One kernel launch samples every row
of a step; the sampled ids come back in one copy. The chain and its order are
the reference's (qwen3_runtime/sampling.py:120-135,250-270); the generator is
counter-based, keyed by (seed, draw index), so a request's tokens do not depend
on what it was batched with. The reference draws from a per-request CPU
generator instead (qwen3_runtime/sampling.py:208-227,293-298).
"""

from __future__ import annotations

from typing import Sequence

import torch

from .params import SamplingParams


class Sampler:
    def __init__(self, ops, slots, vocab_size: int, device):
        self.ops = ops
        self.slots = slots
        self.vocab_size = int(vocab_size)
        self.device = torch.device(device)
        self.fparams = slots.add_tensor("sampler_f32", (8,), torch.float32, survives_restart=True)
        self.iparams = slots.add_tensor("sampler_i32", (2,), torch.int32, survives_restart=True)
        self.seeds = slots.add_tensor("sampler_seed", (2,), torch.int64, survives_restart=True)
        self.counts: torch.Tensor | None = None
        # where sampled ids land on the host: pinned, so that the copy does not wait for the host
        self._landing: torch.Tensor | None = None
        self._landed = torch.cuda.Event() if self.device.type == "cuda" else None

    def admit(self, slot: int, params: SamplingParams, seed: int, prompt: Sequence[int]) -> None:
        """Write the request's options into its slot (zeroed when the slot was taken)."""
        f = torch.tensor(
            [params.temperature, params.top_p, params.min_p, params.repetition_penalty,
             params.presence_penalty, params.frequency_penalty, 0.0, 0.0], dtype=torch.float32)
        self.fparams[slot].copy_(f)
        self.iparams[slot].copy_(torch.tensor([max(0, int(params.top_k)), 0], dtype=torch.int32))
        self.seeds[slot].copy_(torch.tensor([int(seed) & (2**63 - 1), 0], dtype=torch.int64))
        if params.has_penalties():
            if self.counts is None:
                self.counts = self.slots.add_tensor(
                    "sampler_counts", (self.vocab_size,), torch.int32, survives_restart=True)
            ids = torch.tensor(list(prompt), dtype=torch.int32, device=self.device)
            self.ops.count_tokens(self.counts, torch.full_like(ids, slot), ids)

    def sample(self, logits: torch.Tensor, slot_rows: torch.Tensor, reqs) -> tuple[list[int], list[float]]:
        """``logits`` [R, V] float32; ``slot_rows`` int32 [R]; ``reqs`` the R requests in row order."""
        return self.finish(self.launch(logits, slot_rows, reqs))

    def launch(self, logits: torch.Tensor, slot_rows: torch.Tensor, reqs) -> "Drawn":
        """Everything of ``sample`` that the host does not wait for: the kernels, and the copy of
        ids and log-probabilities to host memory. ``Drawn.tokens`` stays on the device, for a
        caller that feeds the next step from there."""
        bias = [(i, t, v) for i, r in enumerate(reqs) for t, v in (r.sampling.logit_bias or {}).items()]
        if bias:
            logits = logits.clone()
            rows = torch.tensor([b[0] for b in bias], dtype=torch.int32, device=self.device)
            toks = torch.tensor([int(b[1]) for b in bias], dtype=torch.int32, device=self.device)
            vals = torch.tensor([float(b[2]) for b in bias], dtype=torch.float32, device=self.device)
            self.ops.add_bias(logits, rows, toks, vals)
        forced = [r.forced_next() for r in reqs]
        any_forced = any(f is not None for f in forced)
        tok, lp, work, both = self.ops.sample(logits, slot_rows, self.fparams, self.iparams, self.seeds,
                                              self.counts, keep_processed=any_forced)
        if any_forced:
            # teacher forcing: the given id, scored under the processed logits
            # (reference: qwen3_runtime/sampling.py:319-325)
            logp = torch.log_softmax(work, dim=-1)
            for i, f in enumerate(forced):
                if f is not None:
                    tok[i] = int(f)
                    lp[i] = logp[i, int(f)]
        if self.counts is not None:
            self.ops.count_tokens(self.counts, slot_rows, tok)
        if both.device.type != "cuda":
            return Drawn(tok, both, None)
        n = both.numel()
        if self._landing is None or self._landing.numel() < n:
            self._landing = torch.empty(max(n, 512), dtype=torch.int32, pin_memory=True)
        host = self._landing[:n].view(both.shape)
        host.copy_(both, non_blocking=True)  # ids and log-probabilities in one copy
        self._landed.record()
        return Drawn(tok, host, self._landed)

    def finish(self, drawn: "Drawn") -> tuple[list[int], list[float]]:
        """Wait for what ``launch`` started (one wait); one ``launch`` is open at a time."""
        if drawn.landed is not None:
            drawn.landed.synchronize()
        host = drawn.host if drawn.landed is not None else drawn.host.cpu()
        return host[0].tolist(), host[1].view(torch.float32).tolist()


class Drawn:
    """A ``Sampler.launch`` under way: the ids on the device, and where they arrive on the host."""

    __slots__ = ("tokens", "host", "landed")

    def __init__(self, tokens, host, landed):
        self.tokens, self.host, self.landed = tokens, host, landed
