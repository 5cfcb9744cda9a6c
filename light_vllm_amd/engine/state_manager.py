"""State slots: one per live sequence of a model whose mixers carry per-sequence state outside the
paged cache (a recurrent state, the tail of a convolution's input). The slot index addresses every
such layer's state tensors. Slots are handed out oldest-free-first and reused without being cleared:
the kernels take a sequence with no context as starting from zeros."""
from __future__ import annotations

from .sequence import Sequence


class StateSlotManager:

    def __init__(self, num_slots: int):
        assert num_slots > 0
        self.num_slots = num_slots
        self._free: dict[int, None] = dict.fromkeys(range(num_slots))
        self.owner: dict[int, int] = {}          # slot -> seq_id

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self, seq: Sequence) -> int:
        assert seq.state_slot < 0, "sequence already owns a state slot"
        slot = next(iter(self._free))            # StopIteration here = no slot free
        del self._free[slot]
        self.owner[slot] = seq.seq_id
        seq.state_slot = slot
        return slot

    def release(self, seq: Sequence) -> None:
        slot = seq.state_slot
        if slot < 0:
            return
        assert self.owner.pop(slot) == seq.seq_id
        self._free[slot] = None
        seq.state_slot = -1
