"""Slots for per-request recurrent state.

Models with recurrent sublayers (state-space scans, short convolutions) keep
a fixed-size state per live request instead of — or beside — KV pages. The
pools are tensors of ``num_slots`` rows owned by the model runner; this class
hands rows out and takes them back. Slot 0 is never handed out: padded lanes
of captured decode graphs read and write it as scratch (the same convention
as KV block 0).

A slot is not cleared when it is reused: the kernels start a sequence whose
first position is 0 from a zero state without reading the slot.
"""

from __future__ import annotations

from typing import Dict, List


class StateSlotManager:
    def __init__(self, num_slots: int):
        if num_slots < 2:
            raise ValueError("need at least one usable slot besides scratch slot 0")
        self.num_slots = num_slots
        self._free: List[int] = list(range(num_slots - 1, 0, -1))
        self._owner: Dict[str, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def has(self, request_id: str) -> bool:
        return request_id in self._owner

    def slot_of(self, request_id: str) -> int:
        return self._owner[request_id]

    def allocate(self, request_id: str) -> int:
        if request_id in self._owner:
            return self._owner[request_id]
        if not self._free:
            raise RuntimeError("Out of state slots")
        slot = self._free.pop()
        self._owner[request_id] = slot
        return slot

    def free(self, request_id: str) -> None:
        slot = self._owner.pop(request_id, None)
        if slot is not None:
            self._free.append(slot)
