"""Slot pool for per-sequence recurrent state (the companion of the paged
block manager for layers that carry a fixed-size state instead of keys).

Accounting only; the state tensors live in ModelRunner. A sequence takes a
slot when it is admitted and keeps it until it finishes, is aborted or is
preempted. Slots are reused without clearing: a sequence whose context
length is 0 starts from a zero state whatever the slot held before.
"""
from __future__ import annotations

from typing import List

from .sequence import Sequence


class StateSlotManager:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free_slots: List[int] = list(range(num_slots - 1, -1, -1))

    @property
    def num_free(self) -> int:
        return len(self.free_slots)

    def can_allocate(self) -> bool:
        return bool(self.free_slots)

    def allocate(self, seq: Sequence) -> int:
        if seq.state_slot >= 0:
            return seq.state_slot
        if not self.free_slots:
            raise RuntimeError("no free recurrent-state slot")
        seq.state_slot = self.free_slots.pop()
        return seq.state_slot

    def free(self, seq: Sequence) -> None:
        if seq.state_slot >= 0:
            self.free_slots.append(seq.state_slot)
            seq.state_slot = -1
