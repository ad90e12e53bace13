"""Slots for per-sequence recurrent state (models whose layers carry a state from token to
token besides, or instead of, a KV cache).  The device tensors live in the runner, one row
per slot in every stateful layer; this is the host-side allocator the scheduler owns next to
the block manager.  A slot's content is never cleared: a sequence that starts at position 0
ignores whatever its slot holds (the kernels start from zeros then), so a slot can go from
one request to the next without any device work.
"""
from __future__ import annotations

from collections import deque


class StateSlotPool:
    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("num_slots must be positive")
        self.num_slots = num_slots
        self._free = deque(range(num_slots))
        self._used = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self) -> int:
        if not self._free:
            raise RuntimeError("no free state slot")
        s = self._free.popleft()
        self._used.add(s)
        return s

    def release(self, slot: int) -> None:
        if slot not in self._used:
            raise ValueError(f"state slot {slot} is not in use")
        self._used.remove(slot)
        self._free.append(slot)          # oldest-freed first: slots rotate
