"""Slots for per-request state of fixed size.

A request gets a slot when it starts and gives it back when it ends; a layer with
state keeps one row per slot on the device and finds its requests' rows through the
step's ``slot_ids``.  (The reference's analogue is the slot index of its per-slot
arrays, ``jllm/engine/runtime.py:23-35``.)  Qwen3 has no such state, the slots are
assigned all the same.
"""
from __future__ import annotations


class OutOfSlots(RuntimeError):
    pass


class StateSlotPool:
    def __init__(self, num_slots: int):
        if num_slots < 1:
            raise ValueError("at least one slot is needed")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))  # lowest slot first
        self._used: set = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> int:
        if not self._free:
            raise OutOfSlots("no free state slot")
        s = self._free.pop()
        self._used.add(s)
        return s

    def release(self, slot: int) -> None:
        if slot not in self._used:
            raise RuntimeError(f"slot {slot} released but not in use")
        self._used.remove(slot)
        self._free.append(slot)
        self._free.sort(reverse=True)
