"""State slots for models with recurrent layers: a request holds one slot (a row of every per-sequence state tensor)
from admission until it ends or is preempted.  Slots are handed out lowest free number first and reused; nothing
is cleared on reuse, because a sequence that starts at position 0 starts from zero state in the kernels."""
from __future__ import annotations

import heapq


class StateSlotManager:
    def __init__(self, num_slots: int):
        if num_slots < 1:
            raise ValueError("need at least one state slot")
        self.num_slots = num_slots
        self._free = list(range(num_slots))
        heapq.heapify(self._free)
        self._held: dict[str, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self) -> bool:
        return bool(self._free)

    def allocate(self, seq_id: str) -> int:
        if seq_id in self._held:
            return self._held[seq_id]
        if not self._free:
            raise ValueError("no free state slot")
        slot = heapq.heappop(self._free)
        self._held[seq_id] = slot
        return slot

    def free(self, seq_id: str) -> None:
        slot = self._held.pop(seq_id, None)
        if slot is not None:
            heapq.heappush(self._free, slot)

    def slot_of(self, seq_id: str) -> int | None:
        return self._held.get(seq_id)
