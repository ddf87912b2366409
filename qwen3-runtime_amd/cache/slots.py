"""Slots for per-request state of fixed size.

A request takes one slot when it is admitted and keeps it until it ends. Any
component may register a tensor with one row per slot: a mixer its recurrent
state, the sampler its draw counter and penalty counts. A slot's rows are
zeroed when the slot is taken. The reference keeps such state on its Python
request object (generator and logprob lists: qwen3_runtime/engine/request.py:64,73-75)
and recounts penalties from the token list each step (qwen3_runtime/sampling.py:57-62).
"""

from __future__ import annotations

from typing import Hashable, Sequence

import torch

from .pages import CacheFull


class StateSlots:
    def __init__(self, num_slots: int, device: torch.device | str = "cpu"):
        if num_slots < 1:
            raise ValueError("num_slots must be positive")
        self.num_slots = int(num_slots)
        self.device = torch.device(device)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._slot_of: dict[Hashable, int] = {}
        self.tensors: dict[str, torch.Tensor] = {}
        self._survives_restart: set[str] = set()

    def add_tensor(self, name: str, shape: Sequence[int], dtype: torch.dtype,
                   survives_restart: bool = False) -> torch.Tensor:
        """One row of ``shape`` per slot. State that follows the tokens in the cache (a mixer's
        recurrence) is zeroed when its request starts over; state that follows the request
        (the sampler's draw counter) survives that: pass ``survives_restart``."""
        if name in self.tensors:
            raise ValueError(f"state tensor {name!r} is registered twice")
        t = torch.zeros((self.num_slots, *shape), dtype=dtype, device=self.device)
        self.tensors[name] = t
        if survives_restart:
            self._survives_restart.add(name)
        return t

    @property
    def num_free(self) -> int:
        return len(self._free)

    def has(self, holder: Hashable) -> bool:
        return holder in self._slot_of

    def slot(self, holder: Hashable) -> int:
        return self._slot_of[holder]

    def take(self, holder: Hashable) -> int:
        if holder in self._slot_of:
            raise AssertionError(f"{holder!r} already holds slot {self._slot_of[holder]}")
        if not self._free:
            raise CacheFull("no free state slot")
        slot = self._free.pop()
        self._slot_of[holder] = slot
        for t in self.tensors.values():
            t[slot].zero_()
        return slot

    def reset(self, holder: Hashable) -> None:
        """The holder starts over from position 0: zero the state that followed its tokens."""
        slot = self._slot_of[holder]
        for name, t in self.tensors.items():
            if name not in self._survives_restart:
                t[slot].zero_()

    def give(self, holder: Hashable) -> None:
        if holder not in self._slot_of:
            raise AssertionError(f"{holder!r} holds no slot")
        self._free.append(self._slot_of.pop(holder))
