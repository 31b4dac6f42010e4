"""State slots for models that carry per-sequence recurrent state.

Paged KV blocks hold what attention layers keep; recurrences, token shifts
and convolution tails keep a fixed-size state per live sequence instead. The
runner allocates every state tensor as [num_slots, ...]; this manager hands a
slot index to a sequence at admission and takes it back when the sequence
finishes, is aborted or is preempted. Slots are reused without clearing: the
kernels start from zero state whenever a run begins at position 0.
"""
from __future__ import annotations


class NoFreeSlots(Exception):
    pass


class StateSlotManager:
    def __init__(self, num_slots: int):
        assert num_slots > 0
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))  # pop() -> lowest first
        self._owner: dict[int, str] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, request_id: str) -> int:
        if not self._free:
            raise NoFreeSlots()
        slot = self._free.pop()
        self._owner[slot] = request_id
        return slot

    def free(self, slot: int) -> None:
        if slot < 0:
            return
        assert slot in self._owner, f"slot {slot} is not allocated"
        del self._owner[slot]
        self._free.append(slot)

    def owner(self, slot: int):
        return self._owner.get(slot)
