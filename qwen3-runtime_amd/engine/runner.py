"""The step function: run the tokens a step brings, from the cache, as one batch.

``ModelRunner.step(entries)`` takes, for each request in the step, its next
tokens and the places whose logits are wanted; it reserves pages, packs the
batch, runs the model once over all tokens of all entries, records the new
lengths and returns float32 logits ``[wanted, vocab]`` in the order of the
entries and of their ``want`` lists. Portions of prompts and single decoded
tokens go through the same pass (the reference's runner may split them into
two forwards: qwen3_runtime/engine/model_runner.py:118-127; its contract is
qwen3_runtime/engine/runner.py:27-41).

Steps that are pure decoding (one token per entry) are replayed from a HIP
graph captured per batch size, with the step's arrays copied into static
buffers first (reference: qwen3_runtime/engine/cuda_graph.py:152-188).
"""

from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from ..cache.pages import CacheFull
from ..parts.base import GroupView, StepContext
from .batch import PackedStep, StepEntry, pack_step


class ModelRunner:
    def __init__(self, model, cache, ops, *, dtype: torch.dtype, device, max_model_len: int | None = None,
                 hip_graph: bool = False):
        self.model = model
        self.cache = cache
        self.ops = ops
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_model_len = int(max_model_len or model.plan.max_positions)
        self.vocab_size = model.plan.vocab_size
        # graphs only where every part of the model can be captured (a part says so itself)
        self.hip_graph = bool(hip_graph) and self.device.type == "cuda" and model.graph_capturable
        self._graphs: dict[tuple, "_DecodeGraph"] = {}
        self._graph_pool = None
        # device copy of the last step's "row_slots" (state slot of each row of the logits)
        self.last_row_slots: torch.Tensor | None = None
        self._pinned: torch.Tensor | None = None
        self._copied = torch.cuda.Event() if self.device.type == "cuda" else None
        self.graph_max_batch = 256
        self.steps_begun = 0
        self._last_graph = None
        # A step may be launched before it is asked for, and then not be asked for after all, only
        # if running it has no effect that a later step could see: keys and values written beyond
        # a request's counted length are such; a per-request state that the step replaces is not.
        self.repeatable = all(s.paged for s in model.plan.caches)
        self.steps_ahead = [0, 0]  # launched before they were asked for; of these, asked for

    # ---- public ------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        self.steps_begun += 1
        self._last_graph = None
        for e in entries:
            end = self.cache.length(e.request_id) + len(e.tokens)
            if end > self.max_model_len:
                raise ValueError(
                    f"request {e.request_id!r} would reach {end} tokens; the limit is {self.max_model_len}"
                )
        try:
            for e in entries:
                self.cache.reserve(e.request_id, len(e.tokens))
        except CacheFull:
            # A replayed decode step takes the pages of the step it expects next while the device
            # runs; if another step comes instead and finds no page, those go back first.
            if not self.cache.trim():
                raise
            for e in entries:
                self.cache.reserve(e.request_id, len(e.tokens))
        pure_decode = all(len(e.tokens) == 1 for e in entries)
        graph = None
        if self.hip_graph and pure_decode and len(entries) <= self.graph_max_batch:
            logits, graph = self._step_graph(entries)
        else:
            packed = pack_step(entries, self.cache, self.vocab_size)
            dev = self._upload(packed)
            self.last_row_slots = dev["row_slots"]
            logits = self._forward(packed, dev)
        for e in entries:
            self.cache.commit(e.request_id, len(e.tokens))
        if graph is not None:
            graph.prepare_next()  # host work for the next step while the GPU runs this one
        self._last_graph = graph
        return logits

    def step_ahead(self, tokens: torch.Tensor) -> bool:
        """The step just run was a replayed decode step, and the caller knows that the next one
        will be the same requests, each with the id that ``tokens`` (int32, on the device, in the
        step's order) holds for it: launch that step now. The next ``step`` must still be called,
        with those ids; it finds its logits computed. Returns whether anything was launched."""
        graph = self._last_graph
        if not self.repeatable or graph is None or not graph.launch_ahead(tokens):
            return False
        self.steps_ahead[0] += 1
        return True

    # ---- eager path ----------------------------------------------------------
    def _upload(self, packed: PackedStep) -> dict[str, torch.Tensor]:
        """All arrays of a step in one host buffer, one copy to the device."""
        sizes = [(name, a.size) for name, a in packed.arrays.items()]
        # keep every array 16-byte aligned on the device
        offsets, total = [], 0
        for _, n in sizes:
            offsets.append(total)
            total += (n + 3) // 4 * 4
        total = max(total, 4)
        if self.device.type == "cuda":
            if self._pinned is None or self._pinned.numel() < total:
                self._pinned = torch.empty(max(total, 1 << 16), dtype=torch.int32, pin_memory=True)
            else:
                self._copied.synchronize()  # the previous step's copy has left the buffer
            host = self._pinned[:total]
        else:
            host = torch.empty(total, dtype=torch.int32)
        host_np = host.numpy()
        for (name, n), off in zip(sizes, offsets):
            host_np[off: off + n] = packed.arrays[name].reshape(-1)
        if self.device.type == "cuda":
            dev = torch.empty(total, dtype=torch.int32, device=self.device)
            dev.copy_(host, non_blocking=True)
            self._copied.record()
        else:
            dev = host.clone()
        out = {}
        for (name, n), off in zip(sizes, offsets):
            out[name] = dev[off: off + n].view(packed.arrays[name].shape)
        return out

    def _context(self, packed: PackedStep, dev: dict[str, torch.Tensor]) -> StepContext:
        groups = [
            GroupView(g.page_size, g.window, dev[f"table{gi}"], dev[f"slots{gi}"])
            for gi, g in enumerate(self.cache.groups)
        ]
        return StepContext(
            ops=self.ops,
            dtype=self.dtype,
            device=self.device,
            num_tokens=packed.num_tokens,
            num_seqs=packed.num_seqs,
            positions=dev["positions"],
            cu_q=dev["cu_q"],
            kv_lens=dev["kv_lens"],
            seq_of_token=dev["seq_of_token"],
            state_slots=dev["state_slots"],
            first_span=dev["first_span"],
            q_lens_host=packed.q_lens,
            kv_lens_host=packed.kv_lens,
            max_q_len=max(packed.q_lens),
            max_kv_len=max(packed.kv_lens),
            groups=groups,
        )

    def _forward(self, packed: PackedStep, dev: dict[str, torch.Tensor]):
        ctx = self._context(packed, dev)
        views = [
            None if st.cache is None else self.cache.view(st.cache, ctx.groups, st.writes_cache)
            for st in self.model.plan.order
        ]
        rows = dev["rows"] if packed.num_rows else None
        with torch.inference_mode():
            return self.model.forward(ctx, dev["ids"], views, rows)

    # ---- graph path ----------------------------------------------------------
    def _step_graph(self, entries: Sequence[StepEntry]):
        from .graph import DecodeGraph

        lens = [self.cache.length(e.request_id) + 1 for e in entries]
        max_kv = max(lens)
        # contexts of very unequal lengths: the ops may cut them another way, which a capture freezes
        unequal = getattr(self.ops, "decode_in_pieces", None)
        key = DecodeGraph.key_for(len(entries), max_kv, all(len(e.want) == 1 for e in entries),
                                  unequal is not None and unequal(lens))
        if key is None:
            packed = pack_step(entries, self.cache, self.vocab_size)
            dev = self._upload(packed)
            self.last_row_slots = dev["row_slots"]
            return self._forward(packed, dev), None
        graph = self._graphs.get(key)
        if graph is None:
            graph = DecodeGraph(self, key)
            self._graphs[key] = graph
        return graph.run(entries), graph
