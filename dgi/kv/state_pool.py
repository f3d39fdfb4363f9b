"""Per-sequence state slots: what a model carries from token to token besides paged keys and values.

A recurrent mixer (Mamba-2) keeps a fixed-size state per sequence, a causal convolution its
last inputs, a bigram embedding the previous token.  None of it grows with the sequence, so it
does not live in pages: the pool owns one tensor ``[num_slots + 1, *shape]`` per named field
(``fields``: name -> (shape, dtype), declared by the model's ``state_fields``), a running
sequence owns one slot index into all of them, and the scheduler hands slots out at admission
and takes them back with the sequence's pages.  Slot 0 is reserved: padded graph rows read and
write it, like page 0 of the block pool.

A slot is NOT cleared when it is handed out.  Every kernel that reads state takes the position
of the first row of the sequence's portion and treats position 0 as "no state yet", so a slot
that another sequence used before is never read by a fresh one.
"""
from __future__ import annotations

import torch


class OutOfSlots(RuntimeError):
    pass


class StatePool:
    def __init__(self, num_slots: int, fields: dict, device="cpu"):
        self.num_slots = int(num_slots)
        self.device = torch.device(device)
        self.fields = {k: (tuple(int(x) for x in sh), dt) for k, (sh, dt) in fields.items()}
        self.tensors = {k: torch.zeros((self.num_slots + 1, *sh), dtype=dt, device=self.device)
                        for k, (sh, dt) in self.fields.items()}
        self._free = list(range(self.num_slots, 0, -1))
        self.stats = {"allocs": 0, "frees": 0}

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.tensors[name]

    @property
    def num_free(self) -> int:
        return len(self._free)

    def slot_bytes(self) -> int:
        return sum(t[0].numel() * t.element_size() for t in self.tensors.values())

    def allocate(self) -> int:
        if not self._free:
            raise OutOfSlots("no free state slot")
        self.stats["allocs"] += 1
        return self._free.pop()

    def free(self, slot: int) -> None:
        if slot <= 0 or slot > self.num_slots or slot in self._free:
            raise RuntimeError(f"bad free of state slot {slot}")
        self._free.append(slot)
        self.stats["frees"] += 1
