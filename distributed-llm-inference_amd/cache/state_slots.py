"""Slots for per-request state of fixed size.

A request takes one slot when it is admitted and gives it back when it ends, is aborted or is
preempted. The slot number indexes device arrays ``[max_slots, ...]`` that hold whatever a part
keeps per request outside the paged cache (a recurrent mixer's state, for instance). The dense
Llama decoder keeps nothing there; the slots exist so that such a part needs no change here.
"""

from __future__ import annotations


class NoFreeSlotError(RuntimeError):
    """Every state slot is taken; nothing was changed."""


class StateSlots:
    def __init__(self, num_slots: int) -> None:
        if num_slots <= 0:
            raise ValueError("num_slots must be positive")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._taken: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise NoFreeSlotError(f"all {self.num_slots} state slots are taken")
        slot = self._free.pop()
        self._taken.add(slot)
        return slot

    def give_back(self, slot: int) -> None:
        if slot not in self._taken:
            raise AssertionError(f"state slot {slot} is given back but not taken")
        self._taken.remove(slot)
        self._free.append(slot)

    def check(self, held: list[int]) -> None:
        assert len(set(held)) == len(held), "a state slot is held twice"
        assert set(held) == self._taken, "taken slots differ from the requests' slots"
        assert len(self._free) + len(self._taken) == self.num_slots, "a state slot is lost"
        assert not set(self._free) & self._taken, "a state slot is both free and taken"
