"""Slots for per-request state of fixed size.

A mixer that carries a state of its own from token to token (rather than, or beside, cached
keys and values) declares its shape; the step function then keeps one tensor [slots, *shape]
per such layer, and every admitted request owns one slot index from this pool until it ends.
A request whose portion starts at position 0 starts from a zeroed slot.  The architecture
built in here declares no state, so its pool is only ever counted, never indexed.
"""

from __future__ import annotations


class StateSlotPool:
    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self.free = list(range(self.num_slots - 1, -1, -1))
        self.owner: dict = {}

    def take(self, key):
        if key in self.owner:
            raise AssertionError(f"{key!r} already owns state slot {self.owner[key]}")
        if not self.free:
            return None
        slot = self.free.pop()
        self.owner[key] = slot
        return slot

    def give(self, key) -> None:
        slot = self.owner.pop(key, None)
        if slot is None:
            raise AssertionError(f"{key!r} owns no state slot")
        self.free.append(slot)

    def slot_of(self, key) -> int:
        return self.owner[key]

    def num_available(self) -> int:
        return len(self.free)

    def check_invariants(self) -> None:
        owned = list(self.owner.values())
        if len(set(owned)) != len(owned) or set(owned) & set(self.free):
            raise AssertionError("a state slot is owned twice or both owned and free")
        if len(owned) + len(self.free) != self.num_slots:
            raise AssertionError("a state slot was lost")
