"""Slots for per-request state of fixed size."""
from __future__ import annotations


class OutOfSlots(RuntimeError):
    pass


class StateSlots:
    """Every live request holds exactly one slot index from admission to
    release.  The index addresses the request's row in every per-request
    device table: the state tensors of mixers that carry state of fixed size
    (one ``[max_seqs, *shape]`` tensor per such layer call) and the sampler's
    per-request counters.  An architecture without such state still takes a
    slot per request, so the mechanism is the same for all.

    The reference has nothing of this kind; the closest are the per-sequence
    flags of LLMSeq (src/core/runtime/BatchManager.h:61-71).
    """

    def __init__(self, max_seqs: int):
        if max_seqs <= 0:
            raise ValueError("at least one slot is needed")
        self.max_seqs = int(max_seqs)
        self._free = list(range(self.max_seqs - 1, -1, -1))
        self._held = [False] * self.max_seqs

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> int:
        if not self._free:
            raise OutOfSlots(f"all {self.max_seqs} request slots are taken")
        s = self._free.pop()
        self._held[s] = True
        return s

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.max_seqs or not self._held[slot]:
            raise ValueError(f"slot {slot} is not held")
        self._held[slot] = False
        self._free.append(slot)

    def check(self) -> None:
        assert len(set(self._free)) == len(self._free)
        assert sum(self._held) + len(self._free) == self.max_seqs
