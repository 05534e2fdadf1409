"""Slots for per-request state of fixed size.

A request gets one slot id when it is admitted and gives it back when it ends; every
run of a layer whose mixer keeps state of its own has a tensor ``[max_slots, *shape]``
indexed by that id.  A slot's state is cleared when the slot is handed out.  Softmax
attention needs none, so for the built-in architecture the tensors dict stays empty and
only the ids are in use (the engine keys per-request sampling state by them).
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch


class OutOfSlots(RuntimeError):
    pass


class StateSlots:
    def __init__(self, max_slots: int) -> None:
        if max_slots < 1:
            raise ValueError("at least one state slot is required")
        self.max_slots = max_slots
        self._free: List[int] = list(range(max_slots - 1, -1, -1))
        self._held = [False] * max_slots
        self.tensors: Dict[int, torch.Tensor] = {}

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def add_state(self, cache_id: int, shape: Tuple[int, ...], dtype: torch.dtype, device) -> torch.Tensor:
        tensor = torch.zeros((self.max_slots, *shape), dtype=dtype, device=device)
        self.tensors[cache_id] = tensor
        return tensor

    def acquire(self) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.max_slots} request slots are in use")
        slot = self._free.pop()
        self._held[slot] = True
        for tensor in self.tensors.values():
            tensor[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.max_slots or not self._held[slot]:
            raise RuntimeError(f"state slot {slot} is not held")
        self._held[slot] = False
        self._free.append(slot)

    def check(self) -> None:
        if len(set(self._free)) != len(self._free):
            raise AssertionError("a state slot is on the free list twice")
        for slot in range(self.max_slots):
            if self._held[slot] == (slot in self._free):
                raise AssertionError(f"state slot {slot} is both free and held, or neither")
