"""Slots for per-request state of fixed size.

A mixer that keeps a fixed-size state per request (the reference has none: its only per-request
device state is KV pages) gets one slot per live request; the slot id travels with the request's
cache handle, is handed to the step function row by row, and is given back when the request ends
or is preempted (the state is then recomputed from the tokens). The allocator exists even when
no mixer of the model asks for state.
"""

from __future__ import annotations


class OutOfStateSlots(RuntimeError):
    pass


class StateSlots:
    def __init__(self, num_slots: int):
        if num_slots < 0:
            raise ValueError("num_slots must be >= 0")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held = [False] * num_slots

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> int:
        if not self._free:
            raise OutOfStateSlots(f"all {self.num_slots} state slots are held")
        s = self._free.pop()
        self._held[s] = True
        return s

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.num_slots:
            raise IndexError(f"state slot {slot} out of range [0, {self.num_slots})")
        if not self._held[slot]:
            raise ValueError(f"state slot {slot} is released twice")
        self._held[slot] = False
        self._free.append(slot)

    def check_invariants(self) -> None:
        assert len(set(self._free)) == len(self._free), "duplicate state slot in free stack"
        assert set(self._free) == {s for s, h in enumerate(self._held) if not h}, "free stack disagrees with held flags"
