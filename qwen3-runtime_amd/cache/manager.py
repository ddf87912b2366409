"""The cache manager: pages and block tables per group of layers, and state slots.

Caches whose ``CacheSpec.group_key()`` is equal form a group: same head
geometry and the same lifetime of keys (all of them, or a window). A group owns
a page pool, a device tensor with the pages of all its caches, and one block
table per request; page ``p`` of a group addresses the same positions in every
cache of the group (reference, for its single group over all layers:
qwen3_runtime/kv/paged.py:24-30). Caches of kind ``"state"`` take no pages:
their tensors live in the state slots.

Lifetime of a request: ``admit`` (slot), then per step ``reserve`` (pages for
the step's tokens; reference: qwen3_runtime/engine/block_manager.py:85-95) and
``commit`` (the tokens are now stored; a window group gives back pages that no
later query can see), finally ``release``. ``restart`` drops the pages but
keeps the slot, for a request that is preempted and recomputed.

Device layout of a paged cache: one tensor per ``PagedStream`` of its spec,
``[page, head, offset, width]`` or, transposed, ``[page, head, width, offset]``.
Keys and values (``"paged_kv"``) are the streams ``k`` and ``v``, the values
transposed inside a page, so that the attention kernels read keys-contiguous
operands for both products; a mixer that keeps something else per token (values of
another width than its keys, one latent vector) names its own streams.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, Sequence

import numpy as np
import torch

from ..parts.base import CacheView, GroupView
from ..parts.plan import CacheSpec
from .pages import CacheFull, PagePool
from .slots import StateSlots


@dataclass
class _Group:
    key: tuple
    spec: CacheSpec
    cache_ids: list[int]
    pool: PagePool
    page_size: int
    window: int | None
    tables: dict[Hashable, list[int]] = field(default_factory=dict)
    # index of the first table entry that still holds a page
    first_live: dict[Hashable, int] = field(default_factory=dict)
    # per stream of the spec: [caches of the group, pages, elements of the stream per page]
    storage: list[torch.Tensor] | None = None

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size if length > 0 else 0


class CacheManager:
    def __init__(
        self,
        specs: Sequence[CacheSpec],
        *,
        page_size: int,
        num_pages: int,
        max_requests: int,
        device: torch.device | str = "cpu",
        dtype: torch.dtype = torch.float32,
        allocate: bool = True,
    ):
        self.specs = list(specs)
        self.page_size = int(page_size)
        self.device = torch.device(device)
        self.dtype = dtype
        self.slots = StateSlots(max_requests, device)
        self.groups: list[_Group] = []
        self._group_of_cache: dict[int, int] = {}
        self._state_of_cache: dict[int, torch.Tensor] = {}
        self._length: dict[Hashable, int] = {}
        self._reserved: dict[Hashable, int] = {}
        # Counts the events after which a block table kept elsewhere no longer describes its
        # request: pages dropped (end, restart) and a request id admitted (possibly again).
        # Whoever keeps a packed copy of tables compares this number before trusting the copy.
        self.epoch = 0
        by_key: dict[tuple, _Group] = {}
        for cid, spec in enumerate(self.specs):
            if spec.paged:
                key = spec.group_key()
                if key not in by_key:
                    by_key[key] = _Group(key, spec, [], PagePool(num_pages), self.page_size, spec.window)
                    self.groups.append(by_key[key])
                by_key[key].cache_ids.append(cid)
                self._group_of_cache[cid] = self.groups.index(by_key[key])
            elif spec.kind == "state":
                dt = dtype if spec.dtype == "model" else getattr(torch, spec.dtype)
                self._state_of_cache[cid] = self.slots.add_tensor(f"cache{cid}", spec.shape, dt)
            else:
                raise ValueError(f"unknown cache kind {spec.kind!r}")
        if allocate:
            for g in self.groups:
                g.storage = [
                    torch.zeros((len(g.cache_ids), g.pool.num_pages, stream.elements_per_token() * self.page_size),
                                dtype=dtype, device=self.device)
                    for stream in g.spec.page_streams()
                ]

    # ---- sizes -------------------------------------------------------------
    @staticmethod
    def bytes_per_page(specs: Sequence[CacheSpec], page_size: int, dtype_bytes: int) -> int:
        """Bytes one page number costs over all paged caches (keys and values).

        4B shape, bfloat16, 16 tokens: 2*36*8*128*2*16 = 2,359,296
        (reference: qwen3_runtime/engine/memory.py:8-14).
        """
        return sum(s.elements_per_token() * page_size * dtype_bytes for s in specs if s.paged)

    def bytes_read(self, kv_lens: Sequence[int], dtype_bytes: int | None = None) -> int:
        """Bytes of cache a step has to read for requests that hold ``kv_lens`` tokens: every
        stream of every paged cache for the tokens a query still sees (all of them, or the
        last ``window``), and every fixed-size state once per request."""
        width = dtype_bytes or torch.finfo(self.dtype).bits // 8
        total = 0
        for spec in self.specs:
            if spec.paged:
                seen = sum(n if spec.window is None else min(n, spec.window) for n in kv_lens)
                total += seen * spec.elements_per_token() * width
        for state in self._state_of_cache.values():
            total += len(kv_lens) * state[0].numel() * state.element_size()
        return total

    @property
    def num_pages(self) -> int:
        return min((g.pool.num_pages for g in self.groups), default=0)

    @property
    def num_free_pages(self) -> int:
        return min((g.pool.num_free for g in self.groups), default=0)

    def pages_needed_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size if length > 0 else 0

    def can_ever_hold(self, length: int) -> tuple[bool, str]:
        """Whether a request that grows to ``length`` tokens fits the pools when it runs alone,
        one token a step if need be: a group that keeps all keys needs the pages of ``length``
        tokens, a window group only the pages its window can touch (it gives the others back as
        it goes). Returns (fits, why not)."""
        for i, g in enumerate(self.groups):
            need = g.pages_for(length)
            if g.window is not None:
                # `window` consecutive positions touch at most this many pages
                need = min(need, (g.window - 1 + g.page_size - 1) // g.page_size + 1)
            if need > g.pool.num_pages:
                what = "" if g.window is None else f" (window {g.window})"
                return False, (f"request length {length} needs {need} cache pages in group {i}{what}; "
                               f"the pool has {g.pool.num_pages}")
        return True, ""

    # ---- request lifetime --------------------------------------------------
    def has(self, rid: Hashable) -> bool:
        return rid in self._length

    def length(self, rid: Hashable) -> int:
        return self._length[rid]

    def admit(self, rid: Hashable) -> int:
        if rid in self._length:
            raise AssertionError(f"request {rid!r} is admitted twice")
        slot = self.slots.take(rid)
        self.epoch += 1
        self._length[rid] = 0
        self._reserved[rid] = 0
        for g in self.groups:
            g.tables[rid] = []
            g.first_live[rid] = 0
        return slot

    def max_reservable_tokens(self, rid: Hashable, limit: int) -> int:
        """Largest ``n <= limit`` whose pages fit in held plus free pages of every group
        (reference: qwen3_runtime/engine/block_manager.py:74-83)."""
        if limit <= 0:
            return 0
        start = self._length[rid]
        n = limit
        for g in self.groups:
            capacity = (len(g.tables[rid]) + g.pool.num_free) * g.page_size
            n = min(n, capacity - start)
        return max(0, n)

    def reserve(self, rid: Hashable, num_tokens: int) -> None:
        """Take the pages that ``num_tokens`` more tokens need, in every group, or none."""
        if num_tokens < 0:
            raise ValueError("num_tokens must be non-negative")
        end = self._length[rid] + num_tokens
        for g in self.groups:
            if g.pages_for(end) - len(g.tables[rid]) > g.pool.num_free:
                raise CacheFull(
                    f"cache pool exhausted: request {rid!r} needs "
                    f"{g.pages_for(end) - len(g.tables[rid])} more pages, {g.pool.num_free} are free"
                )
        for g in self.groups:
            table = g.tables[rid]
            while len(table) < g.pages_for(end):
                table.append(g.pool.take(rid))
        self._reserved[rid] = max(self._reserved[rid], end)

    def trim(self) -> int:
        """Give back every page that a request holds only for tokens it has reserved and not
        stored (pages taken ahead for a step that then was not the next one). Returns how many
        went back; tables that were handed out before are void then, as after any loss of pages."""
        returned = 0
        for rid, length in self._length.items():
            if self._reserved[rid] <= length:
                continue
            for g in self.groups:
                table = g.tables[rid]
                while len(table) > g.pages_for(length):
                    page = table.pop()
                    if page >= 0:
                        g.pool.give(page, rid)
                        returned += 1
            self._reserved[rid] = length
        if returned:
            self.epoch += 1
        return returned

    def commit(self, rid: Hashable, num_tokens: int) -> None:
        """``num_tokens`` more tokens are stored. Window groups give back what no query sees."""
        new_len = self._length[rid] + num_tokens
        if new_len > self._reserved[rid]:
            raise AssertionError(f"request {rid!r} stored {new_len} tokens but reserved {self._reserved[rid]}")
        self._length[rid] = new_len
        for g in self.groups:
            if g.window is None:
                continue
            # the next query sits at position >= new_len and sees keys > its position - window
            first_needed = new_len - g.window + 1
            table = g.tables[rid]
            i = g.first_live[rid]
            while i < len(table) and (i + 1) * g.page_size <= first_needed:
                g.pool.give(table[i], rid)
                table[i] = -1
                i += 1
            g.first_live[rid] = i

    def _drop_pages(self, rid: Hashable) -> None:
        self.epoch += 1
        for g in self.groups:
            for page in g.tables[rid]:
                if page >= 0:
                    g.pool.give(page, rid)
            g.tables[rid] = []
            g.first_live[rid] = 0
        self._length[rid] = 0
        self._reserved[rid] = 0

    def restart(self, rid: Hashable) -> None:
        """Give back all pages and zero the state; the request will be computed again from 0."""
        self._drop_pages(rid)
        self.slots.reset(rid)

    def release(self, rid: Hashable) -> None:
        self._drop_pages(rid)
        for g in self.groups:
            del g.tables[rid], g.first_live[rid]
        del self._length[rid], self._reserved[rid]
        self.slots.give(rid)

    def live_requests(self) -> list[Hashable]:
        return list(self._length)

    def check(self) -> None:
        """Invariants: no page lost, none held twice, tables agree with the pools."""
        for g in self.groups:
            g.pool.check()
            held = [p for t in g.tables.values() for p in t if p >= 0]
            if len(set(held)) != len(held):
                raise AssertionError("a page stands in two block tables")
            if len(held) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError(
                    f"{g.pool.num_pages - g.pool.num_free - len(held)} pages are neither free nor in a table"
                )
            for rid, table in g.tables.items():
                for p in table:
                    if p >= 0 and g.pool.holder_of(p) != rid:
                        raise AssertionError(f"page {p} in {rid!r}'s table is held by {g.pool.holder_of(p)!r}")

    # ---- what a step reads -------------------------------------------------
    def block_table(self, group: int, rid: Hashable) -> list[int]:
        return self.groups[group].tables[rid]

    def table_width(self, rids: Sequence[Hashable]) -> int:
        return max((len(g.tables[r]) for g in self.groups for r in rids), default=1) or 1

    def fill_tables(self, group: int, rids: Sequence[Hashable], out: np.ndarray) -> None:
        """Write the requests' block tables into ``out`` [S, W] int32, -1 where no page."""
        out.fill(-1)
        g = self.groups[group]
        for row, rid in enumerate(rids):
            table = g.tables[rid]
            out[row, : len(table)] = table

    def token_slots(self, group: int, rid: Hashable, start: int, n: int) -> np.ndarray:
        """``page * page_size + offset`` of positions ``start .. start+n-1``
        (reference: qwen3_runtime/engine/block_manager.py:264-270)."""
        g = self.groups[group]
        if n == 1:  # a decoded token: no arrays needed
            page = g.tables[rid][start // g.page_size]
            if page < 0:
                raise AssertionError(f"request {rid!r} writes to a position whose page was given back")
            return np.asarray([page * g.page_size + start % g.page_size], dtype=np.int32)
        pos = np.arange(start, start + n, dtype=np.int64)
        table = np.asarray(g.tables[rid], dtype=np.int64)
        pages = table[pos // g.page_size]
        if (pages < 0).any():
            raise AssertionError(f"request {rid!r} writes to a position whose page was given back")
        return (pages * g.page_size + pos % g.page_size).astype(np.int32)

    def group_of_cache(self, cache_id: int) -> int | None:
        return self._group_of_cache.get(cache_id)

    def view(self, cache_id: int, group_views: Sequence[GroupView], writes: bool = True) -> CacheView:
        spec = self.specs[cache_id]
        if spec.kind == "state":
            return CacheView(spec, writes=writes, state=self._state_of_cache[cache_id])
        gi = self._group_of_cache[cache_id]
        g = self.groups[gi]
        i = g.cache_ids.index(cache_id)
        n = g.pool.num_pages
        pages = {stream.name: store[i].view(n, *stream.page_shape(g.page_size))
                 for stream, store in zip(spec.page_streams(), g.storage)}
        return CacheView(spec, writes=writes, group=group_views[gi], k=pages.get("k"), v=pages.get("v"), pages=pages)
