"""Slots for per-request state of fixed size.  A slot id is what a batch row refers to; a mixer whose state
does not grow with the sequence keeps it at `state[slot]`.  Slots are handed out like pages: a stack, so a
freed slot is the next one taken.

`SlotArrays` is what every request keeps on the device between steps whatever its mixers are: `SLOT_WORDS` 32-bit
words (tokens held, the token chosen last, temperature, seed, draws made so far, whether the slot is taken) and one
row of each cache group's block table.  The reference keeps all of this in Python objects and uploads the tables once
per layer and step (ampere_kv/scheduler.py:14-34, ampere_kv/runner.py:207-213); here a step uploads only what changed -
the table entries of pages that were handed out or given back - and the sampler reads and advances a request's
sampling state where it lies."""

from __future__ import annotations

import struct

import torch

SLOT_WORDS = 8
WORD_LENGTH, WORD_LAST_TOKEN, WORD_TEMPERATURE, WORD_SEED_LOW, WORD_SEED_HIGH, WORD_DRAWS, WORD_TAKEN = range(7)
NO_TOKEN = -1


class SlotArrays:
    """One int32 tensor on the device: `[slots, SLOT_WORDS]` words, then per cache group `[slots, table_width]` page
    ids.  `words` and `tables[g]` are views of it; an offset into the whole is what a step's patches name."""

    def __init__(self, num_slots: int, num_groups: int, table_width: int, device):
        self.num_slots, self.num_groups, self.table_width = num_slots, num_groups, table_width
        self.device = torch.device(device)
        size = num_slots * SLOT_WORDS + num_groups * num_slots * table_width
        self.state = torch.zeros(size, dtype=torch.int32, device=self.device)
        self.words = self.state[:num_slots * SLOT_WORDS].view(num_slots, SLOT_WORDS)
        self.tables = []
        for group in range(num_groups):
            first = self.table_offset(group, 0, 0)
            self.tables.append(self.state[first:first + num_slots * table_width].view(num_slots, table_width))
            self.tables[-1].fill_(-1)
        self.words[:, WORD_LAST_TOKEN] = NO_TOKEN

    def table_offset(self, group: int, slot: int, index: int) -> int:
        return self.num_slots * SLOT_WORDS + (group * self.num_slots + slot) * self.table_width + index

    def take(self, slot: int, temperature: float, seed: int) -> None:
        """A request takes the slot: its words start fresh (nothing held, no token chosen, no draw made, the request's
        own temperature and seed) and its table rows name no page.  One small copy per request, not per step."""
        bits = struct.unpack("<i", struct.pack("<f", float(temperature)))[0]
        low, high = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
        signed = lambda word: word - (1 << 32) if word >= (1 << 31) else word
        fresh = torch.tensor([0, NO_TOKEN, bits, signed(low), signed(high), 0, 1, 0], dtype=torch.int32)
        if self.device.type == "cuda":
            # pinned memory from torch's caching host allocator, which keeps it until the copy has been made
            self.words[slot].copy_(fresh.pin_memory(), non_blocking=True)
        else:
            self.words[slot].copy_(fresh)
        for table in self.tables:
            table[slot].fill_(-1)

    def write_row(self, group: int, slot: int, pages) -> None:
        """The whole row of a request's block table at once (`pages`: its int32 page ids from entry 0 on) - for tokens
        that were registered outside a step, too many for a step's list of changes."""
        row = torch.from_numpy(pages.copy())
        if self.device.type == "cuda":
            row = row.pin_memory()
        self.tables[group][slot, :row.shape[0]].copy_(row, non_blocking=True)

    def give_back(self, slot: int) -> None:
        self.words[slot, WORD_TAKEN] = 0


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
