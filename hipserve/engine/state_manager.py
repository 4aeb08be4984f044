"""Per-sequence state slots for models with recurrent layers: the sequence-level view
of the device state tensors (``model.allocate_state``), beside the paged-cache block
manager. A sequence holds one slot from admission until it finishes, is aborted or is
preempted; the slot indexes every recurrent layer's ``[slots, width]`` state. A step
that starts a sequence at position 0 starts from a zero state, whatever a previous
owner left in the slot."""
from __future__ import annotations

from .request import Sequence


class StateSlots:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))

    def num_free(self) -> int:
        return len(self._free)

    def can_allocate(self, seq: Sequence) -> bool:
        return seq.state_slot is not None or bool(self._free)

    def allocate(self, seq: Sequence) -> int:
        if seq.state_slot is None:
            if not self._free:
                raise RuntimeError("no free state slot")
            seq.state_slot = self._free.pop()
        return seq.state_slot

    def free(self, seq: Sequence):
        if seq.state_slot is not None:
            self._free.append(seq.state_slot)
            seq.state_slot = None
