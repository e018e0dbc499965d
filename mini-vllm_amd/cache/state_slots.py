"""Slots for per-request state of fixed size (what a recurrent mixer would carry from token to
token). A request takes one slot index when it is admitted and gives it back when it ends or
is preempted; the index addresses row ``slot`` of every stateful call's state tensor. The
reference has no such state; the Qwen3 plan asks for zero bytes per slot, but the slot index is
allocated, carried through the step and released all the same."""
from __future__ import annotations

from collections import deque
from typing import Deque, Set


class OutOfSlots(RuntimeError):
    pass


class StateSlots:
    def __init__(self, num_slots: int):
        if num_slots < 1:
            raise ValueError(f"need at least one state slot, got {num_slots}")
        self.num_slots = num_slots
        self._free: Deque[int] = deque(range(num_slots))
        self._used: Set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self) -> int:
        if not self._free:
            raise OutOfSlots("no free state slot")
        s = self._free.popleft()
        self._used.add(s)
        return s

    def release(self, slot: int) -> None:
        if slot not in self._used:
            raise AssertionError(f"state slot {slot} is released but not held")
        self._used.remove(slot)
        self._free.append(slot)

    def check(self) -> None:
        assert len(self._free) + len(self._used) == self.num_slots
        assert not (set(self._free) & self._used)
