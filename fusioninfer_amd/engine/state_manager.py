"""State-slot manager: fixed-size per-sequence state for recurrent mixers.

Paged blocks hold what grows with a sequence (keys/values); a recurrent
mixer instead needs a constant-size state per live sequence (the delta
rule's matrix, the previous token's hidden vector for a token shift).
Those live in slot-indexed device tensors owned by the model runner; this
manager hands slot ids to sequences and takes them back, next to the
BlockManager.

A slot is NOT cleared when it is handed out: the kernels start from a zero
state whenever a sequence's chunk begins at position 0, so a reused slot
cannot leak its previous owner's state and re-prefill after preemption is
exact.
"""

from __future__ import annotations

from typing import Dict, List

from fusioninfer_amd.engine.sequence import Sequence


class StateSlotManager:
    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        # pop() takes from the end: lowest ids first, most recently freed
        # slot is reused first
        self.free_slots: List[int] = list(range(num_slots - 1, -1, -1))
        self.owner: Dict[int, str] = {}

    def num_free(self) -> int:
        return len(self.free_slots)

    def can_allocate(self) -> bool:
        return bool(self.free_slots)

    def allocate(self, seq: Sequence) -> int:
        assert seq.state_slot < 0, f"{seq.seq_id} already holds a slot"
        if not self.free_slots:
            raise RuntimeError("no free state slot")
        slot = self.free_slots.pop()
        self.owner[slot] = seq.seq_id
        seq.state_slot = slot
        return slot

    def free(self, seq: Sequence) -> None:
        slot = seq.state_slot
        if slot < 0:
            return
        assert self.owner.get(slot) == seq.seq_id, (slot, seq.seq_id)
        del self.owner[slot]
        self.free_slots.append(slot)
        seq.state_slot = -1
