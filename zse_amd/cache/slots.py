"""Slots of fixed size for per-request state.

The reference keeps no such state (only bookkeeping dictionaries,
cache/cache_manager.py:130-133).  A slot is where a mixer whose memory does not
grow with the sequence keeps it; every live request owns exactly one, given at
admission and returned with its pages.  The bytes of a slot are laid out by
the model: each cache-owning entry of the execution order with a fixed-size
need gets a range of its own.
"""
from __future__ import annotations

from typing import Dict, List


class OutOfSlots(RuntimeError):
    pass


class StateSlots:
    def __init__(self, num_slots: int, slot_bytes: int):
        if num_slots <= 0:
            raise ValueError("need at least one slot")
        self.num_slots = int(num_slots)
        self.slot_bytes = int(slot_bytes)
        self._free: List[int] = list(range(self.num_slots - 1, -1, -1))
        self._of: Dict[object, int] = {}

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def acquire(self, owner) -> int:
        if owner in self._of:
            raise ValueError(f"{owner!r} already holds slot {self._of[owner]}")
        if not self._free:
            raise OutOfSlots(f"all {self.num_slots} slots are in use")
        s = self._free.pop()
        self._of[owner] = s
        return s

    def release(self, owner) -> None:
        s = self._of.pop(owner, None)
        if s is not None:
            self._free.append(s)

    def slot_of(self, owner) -> int:
        return self._of[owner]

    def holders(self):
        return dict(self._of)

    def check(self) -> None:
        used = list(self._of.values())
        if len(set(used)) != len(used) or set(used) & set(self._free) or \
                len(used) + len(self._free) != self.num_slots or len(set(self._free)) != len(self._free):
            raise AssertionError("slot bookkeeping is inconsistent")
