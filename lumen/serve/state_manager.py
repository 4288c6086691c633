"""Recurrent-state slots of hybrid models (the counterpart of BlockManager for state that does
not grow with the sequence).

A running sequence of a model with recurrent or convolutional layers owns ONE slot of the
runner's state tensors ([slots, ...] per layer) from admission until it finishes, is aborted or
is preempted.  Slots are handed out lowest-free-first and reused without being cleared: the
kernels treat a segment that starts at position 0 as starting from zero state, so a new owner
(or a preempted sequence recomputed from its first token) never sees the previous one's state.
"""
from __future__ import annotations

import heapq
from typing import Dict, List


class NoFreeSlots(RuntimeError):
    pass


class StateSlots:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free: List[int] = list(range(num_slots))
        heapq.heapify(self.free)
        self.owner: Dict[int, int] = {}      # seq_id -> slot

    @property
    def num_free(self) -> int:
        return len(self.free)

    def alloc(self, seq_id: int) -> int:
        s = self.owner.get(seq_id)
        if s is not None:
            return s
        if not self.free:
            raise NoFreeSlots(f"all {self.num_slots} state slots are in use")
        s = heapq.heappop(self.free)
        self.owner[seq_id] = s
        return s

    def slot(self, seq_id: int) -> int:
        return self.owner[seq_id]

    def release(self, seq_id: int) -> None:
        s = self.owner.pop(seq_id, None)
        if s is not None:
            heapq.heappush(self.free, s)
