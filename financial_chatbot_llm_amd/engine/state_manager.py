"""Recurrent-state slots: one fixed-size state record per running sequence.

Models with recurrent layers (state-space mixers) keep, per sequence, a small f32 state next to the
paged cache.  The records live in per-layer arrays indexed by a slot id; this pool hands the ids
out.  A sequence takes a slot when it is admitted and gives it back when it finishes, is aborted or
is preempted (it then recomputes from position 0, which re-initialises whatever slot it gets).
Slots are not cleared on reuse: the kernels start a sequence's first segment from zero state.
"""
from __future__ import annotations

from typing import List

from .sequence import Sequence


class StateSlotPool:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free_list: List[int] = list(range(num_slots - 1, -1, -1))
        self.reuses = 0                      # slots handed out again after a release
        self._used_once = [False] * num_slots

    def num_free(self) -> int:
        return len(self.free_list)

    def acquire(self, seq: Sequence) -> bool:
        """Give ``seq`` a slot (True), or report that none is free (False).  Idempotent."""
        if seq.state_slot >= 0:
            return True
        if not self.free_list:
            return False
        s = self.free_list.pop()
        if self._used_once[s]:
            self.reuses += 1
        self._used_once[s] = True
        seq.state_slot = s
        return True

    def release(self, seq: Sequence) -> None:
        if seq.state_slot >= 0:
            self.free_list.append(seq.state_slot)
            seq.state_slot = -1
