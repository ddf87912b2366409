"""Pure-decode steps replayed from captured HIP graphs.

A graph is captured per (batch size, bucket of the longest context, whether the
contexts are of very unequal lengths: the attention kernel then cuts them another way). Its
kernels read the step's arrays (token ids, positions, lengths, block tables,
slots) from one static device buffer; a replay fills that buffer with one copy
and launches the whole step at once, which removes the per-kernel launch cost
that otherwise exceeds the time the kernels need at small batch
(reference, same idea per batch size: qwen3_runtime/engine/cuda_graph.py:82-104,152-188).
The bucket fixes what a capture freezes: the width of the block table and the
number of key splits of the attention kernel. Nothing that clears memory with
a memset node is recorded.
"""

from __future__ import annotations

import gc
from typing import Sequence

import numpy as np
import torch

from ..cache.pages import CacheFull
from .batch import StepEntry, pack_step

MIN_BUCKET = 512


class DecodeGraph:
    @staticmethod
    def key_for(batch: int, max_kv: int, all_want: bool, unequal: bool = False):
        if not all_want:
            return None
        bucket = MIN_BUCKET
        while bucket < max_kv:
            bucket *= 2
        return (batch, bucket, bool(unequal))

    def __init__(self, runner, key):
        self.runner = runner
        self.batch, self.bucket, self.unequal = key
        cache = runner.cache
        self.width = max(1, -(-self.bucket // cache.page_size))
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits = None
        self.layout: list[tuple[str, int, tuple]] | None = None
        self.host = self.dev = None
        self.copied = torch.cuda.Event()
        self.ctx = None
        self.runs = 0
        # what the host buffer holds: the requests of the last fill and their lengths before it
        self._last_rids: list | None = None
        self._last_starts: list[int] | None = None
        self._last_epoch = -1  # the cache's epoch at the last fill: a later one voids the buffer
        self._host_views = None
        self._row_index = None
        self._prepared = False  # the host buffer holds the step after the one launched last
        self._ahead = None      # (requests, lengths, epoch) of a step launched before it was asked for
        # the ids that step was fed, brought to the host beside it: the step asked for must bring the same
        self._ahead_ids: torch.Tensor | None = None
        self._ahead_ids_here = torch.cuda.Event()

    def _fill(self, entries: Sequence[StepEntry]):
        runner = self.runner
        rids = [e.request_id for e in entries]
        starts = [runner.cache.length(r) for r in rids]
        # The kept buffer is only good while no request has dropped pages or been admitted since:
        # the same id at the same length may by then own other pages (restart after preemption,
        # release and a new request under the old id).
        if self.graph is not None and rids == self._last_rids and runner.cache.epoch == self._last_epoch:
            if starts != self._last_starts and all(a == b + 1 for a, b in zip(starts, self._last_starts)):
                self._advance(rids, starts)
            if starts == self._last_starts:  # the buffer holds this step, but for the ids
                self._send(entries)
                return None
        self._last_rids, self._last_starts, self._last_epoch = rids, starts, runner.cache.epoch
        packed = pack_step(entries, runner.cache, runner.vocab_size, table_width=self.width)
        if self.layout is None:
            off, layout = 0, []
            for name, a in packed.arrays.items():
                layout.append((name, off, a.shape))
                off += (a.size + 3) // 4 * 4
            self.layout, total = layout, max(off, 4)
            self.host = torch.empty(total, dtype=torch.int32, pin_memory=True)
            self.dev = torch.zeros(total, dtype=torch.int32, device=runner.device)
        else:
            self.copied.synchronize()  # the previous copy has left the host buffer
        host = self.host.numpy()
        for name, off, shape in self.layout:
            a = packed.arrays[name]
            if a.shape != shape:
                raise AssertionError(f"decode graph: array {name} changed shape {shape} -> {a.shape}")
            host[off: off + a.size] = a.reshape(-1)
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        return packed

    def _host(self):
        if self._host_views is None:
            host = self.host.numpy()
            self._host_views = {name: host[off: off + int(np.prod(shape))].reshape(shape)
                                for name, off, shape in self.layout}
            self._row_index = np.arange(self.batch)
        return self._host_views

    def _advance(self, rids, starts) -> None:
        """The same requests one token further (the usual decode step): the host buffer is brought
        up to date in place, but for the ids. Positions and lengths one up, the slots of the new
        positions, and a block-table entry where a request has begun a page; groups with a window
        (whose pages are given back as the window passes) get their tables written afresh. The
        pages of the new positions must be reserved."""
        cache = self.runner.cache
        self.copied.synchronize()  # the previous copy has left the host buffer
        view = self._host()
        pos = np.asarray(starts, dtype=np.int64)
        view["positions"][:] = pos
        view["kv_lens"][:] = pos + 1
        for gi, g in enumerate(cache.groups):
            table = view[f"table{gi}"]
            page_index = pos // g.page_size
            if g.window is not None:
                cache.fill_tables(gi, rids, table)
            else:
                for i in np.nonzero(pos % g.page_size == 0)[0]:
                    table[i, page_index[i]] = g.tables[rids[i]][page_index[i]]
            pages = table[self._row_index, page_index].astype(np.int64)
            if (pages < 0).any():
                raise AssertionError("a request writes to a position whose page was given back")
            view[f"slots{gi}"][:] = pages * g.page_size + pos % g.page_size
        self._last_starts = list(starts)

    def _send(self, entries: Sequence[StepEntry]) -> None:
        """Write the step's ids into the host buffer and start its copy to the device."""
        ids = np.asarray([e.tokens[0] for e in entries], dtype=np.int64)
        if ids.min() < 0 or ids.max() >= self.runner.vocab_size:
            raise ValueError(f"token id outside [0, {self.runner.vocab_size})")
        self._host()["ids"][:] = ids
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def prepare_next(self) -> None:
        """Called when the step just launched has been entered into the cache's books: while the
        GPU runs it, get the buffer ready for the step that most often follows, the same requests
        one token further. Their pages are reserved now, in the order the scheduler would; if one
        cannot get its page, or would leave this graph's bucket, nothing is prepared. A request
        that ends instead gives its page back with all its others."""
        if self.graph is None or self._last_rids is None:
            return
        cache, rids = self.runner.cache, self._last_rids
        if cache.epoch != self._last_epoch or not all(cache.has(r) for r in rids):
            return
        starts = [cache.length(r) for r in rids]
        if any(a != b + 1 for a, b in zip(starts, self._last_starts)):
            return
        if max(starts) + 1 > min(self.bucket, self.runner.max_model_len):
            return
        try:
            for r in rids:
                cache.reserve(r, 1)
        except CacheFull:
            return
        self._advance(rids, starts)
        self._prepared = True

    def launch_ahead(self, tokens: torch.Tensor) -> bool:
        """Launch the step that ``prepare_next`` has prepared, now, with the ids that the sampler
        has just written on the device (int32 [batch], in the step's order), before the host has
        seen them. The caller knows that the step will be asked for: no request ends with these
        ids, and nobody else waits. ``run`` then finds its work done. If something else is asked
        for instead (a request added or cancelled in between), the launch has only written keys
        and values at positions that the cache's books do not count, into pages reserved for
        them; whoever owns such a page later writes a position before reading it."""
        if not self._prepared or self.graph is None:
            return False
        if tokens.shape != (self.batch,) or tokens.dtype != torch.int32 or tokens.device != self.dev.device:
            raise ValueError(f"ids for the step ahead: int32 [{self.batch}] on {self.dev.device} expected")
        self._prepared = False
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        self.views_dev["ids"].copy_(tokens)
        if self._ahead_ids is None:
            self._ahead_ids = torch.empty(self.batch, dtype=torch.int32, pin_memory=True)
        self._ahead_ids.copy_(tokens, non_blocking=True)  # a few bytes, on their way before the step's kernels
        self._ahead_ids_here.record()
        self.runner.last_row_slots = self.views_dev["row_slots"]
        self.graph.replay()
        self._ahead = (list(self._last_rids), list(self._last_starts), self._last_epoch, self.runner.steps_begun)
        return True

    def _views(self):
        return {name: self.dev[off: off + int(np.prod(shape))].view(shape) for name, off, shape in self.layout}

    def run(self, entries: Sequence[StepEntry]):
        runner = self.runner
        ahead, self._ahead = self._ahead, None
        self._prepared = False
        if ahead is not None:
            rids = [e.request_id for e in entries]
            # the very next step of the runner (no other has used the graphs' shared memory since),
            # for the same requests at the same lengths, owning the same pages
            if ahead == (rids, [runner.cache.length(r) for r in rids], runner.cache.epoch, runner.steps_begun - 1):
                # ... and fed the ids these entries bring (they came to the host beside the launch;
                # whoever waited for the sampled ids has waited for these too). Other ids: the
                # launched step is one nobody asked for, and this one runs as any other.
                self._ahead_ids_here.synchronize()
                if self._ahead_ids.tolist() == [e.tokens[0] for e in entries]:
                    runner.last_row_slots = self.views_dev["row_slots"]
                    runner.steps_ahead[1] += 1
                    return self.logits
        packed = self._fill(entries)
        if self.graph is None:
            if self.ctx is None:
                self.views_dev = self._views()
                packed.kv_lens = [self.bucket] * self.batch  # launch shapes are those of the bucket
                self.ctx = runner._context(packed, self.views_dev)
                # the bucket's length, not the batch's, now fixes every launch shape (key splits too);
                # where the lengths are very unequal the attention kernel is told them as they are
                # now, to choose the length of its pieces by
                if self.unequal:
                    self.ctx.scratch["attn_lens"] = [runner.cache.length(e.request_id) + 1 for e in entries]
                self.cache_views = [
                    None if st.cache is None else runner.cache.view(st.cache, self.ctx.groups, st.writes_cache)
                    for st in runner.model.plan.order
                ]
            dev = self.views_dev
            runner.last_row_slots = dev["row_slots"]
            self.runs += 1
            with torch.inference_mode():
                if self.runs < 2:
                    # the first call at this size runs eagerly: it fills the attention work list
                    # and warms the allocator; the capture happens on the second call
                    return runner.model.forward(self.ctx, dev["ids"], self.cache_views, dev["rows"])
                graph = torch.cuda.CUDAGraph()
                torch.cuda.synchronize(runner.device)
                # all graphs of a runner take their buffers from one pool: only one of them runs
                # at a time and its logits are consumed before the next step, so the memory they
                # need is that of the largest, not the sum over batch sizes and buckets
                if runner._graph_pool is None:
                    runner._graph_pool = torch.cuda.graph_pool_handle()
                # Graphs of an engine that was dropped earlier may still wait for the collector of
                # reference cycles; destroying a graph is not allowed while a stream captures, and
                # the error is raised in a destructor, which ends the process. So the collector
                # does not run inside the capture. (A full collection before every capture would
                # do as well, and cost 15 % of a continuous-batching run that captures a graph
                # for every batch size it passes through.)
                collecting = gc.isenabled()
                gc.disable()
                try:
                    with torch.cuda.graph(graph, pool=runner._graph_pool):
                        self.logits = runner.model.forward(self.ctx, dev["ids"], self.cache_views, dev["rows"])
                finally:
                    if collecting:
                        gc.enable()
                self.graph = graph
        runner.last_row_slots = self.views_dev["row_slots"]
        self.graph.replay()
        return self.logits

    def _min_kv_heads(self) -> int:
        heads = [stream.heads for s in self.runner.model.plan.caches for stream in s.page_streams()]
        return min(heads) if heads else 1
