"""Slots for per-request state of fixed size.  A slot id is what a batch row refers to; a mixer whose state
does not grow with the sequence keeps it at `state[slot]`.  Slots are handed out like pages: a stack, so a
freed slot is the next one taken."""

from __future__ import annotations


class SlotsExhausted(RuntimeError):
    pass


class SlotTable:
    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("at least one slot is needed")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise SlotsExhausted("every request slot is taken")
        slot = self._free.pop()
        self._held[slot] = True
        return slot

    def give_back(self, slot: int) -> None:
        if not (0 <= slot < self.num_slots) or not self._held[slot]:
            raise ValueError(f"slot {slot} is not taken")
        self._held[slot] = False
        self._free.append(slot)
