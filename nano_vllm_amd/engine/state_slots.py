"""Slots for per-sequence state of stateful layers (recurrent state, convolution tails), beside the paged KV cache.

A slot is an index into every stateful layer's state tensors `[num_slots, ...]` (engine/runner.py allocates them). A
sequence takes a slot when it is admitted and gives it back when it finishes or is preempted; freed slots are handed out
again lowest first and are NOT cleared: the kernels start a sequence whose first token is position 0 from zeros whatever
its slot holds. A preempted sequence is recomputed from its first token, as its pages are.
"""
from __future__ import annotations

import heapq


class StateSlotManager:

    def __init__(self, num_slots: int):
        assert num_slots > 0
        self.num_slots = num_slots
        self._free = list(range(num_slots))          # a heap: lowest free slot first
        self._owner: dict[int, int] = {}             # slot -> seq_id

    @property
    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self) -> bool:
        return bool(self._free)

    def allocate(self, seq) -> int:
        assert seq.state_slot < 0, "sequence already holds a state slot"
        slot = heapq.heappop(self._free)
        self._owner[slot] = seq.seq_id
        seq.state_slot = slot
        return slot

    def release(self, seq) -> None:
        slot = seq.state_slot
        if slot < 0:
            return
        assert self._owner.pop(slot) == seq.seq_id
        heapq.heappush(self._free, slot)
        seq.state_slot = -1
