"""Slot-addressed recurrent state for models whose mixers carry state from
token to token (matrix memories, convolution tails, shifted inputs).

A running sequence owns one slot for its whole life; every state-bearing
layer keeps one fp32 tensor [num_slots, ...] per state kind, indexed by that
slot. Kernels load a slot's state at the start of a step's portion and
store it at the end. A portion that starts at position 0 starts from zero
state whatever the slot holds, so slots are handed out again without
clearing - a preempted sequence that restarts from its first token, or a
new sequence in a used slot, never sees old state.

Sized for 288 GB HBM: state is small next to the paged cache (a 64x128x128
fp32 memory is 4 MiB per layer and slot), so the pool simply holds
max_num_seqs slots.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch


class SlotAllocator:
    """Free-list of state slots (lowest free slot first)."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self.free: List[int] = list(range(num_slots))
        self.owner: List[Optional[str]] = [None] * num_slots

    @property
    def num_free(self) -> int:
        return len(self.free)

    def alloc(self, owner: Optional[str] = None) -> Optional[int]:
        if not self.free:
            return None
        slot = self.free.pop(0)
        self.owner[slot] = owner
        return slot

    def release(self, slot: int):
        assert 0 <= slot < self.num_slots and slot not in self.free
        self.owner[slot] = None
        self.free.append(slot)
        self.free.sort()

    def clear(self):
        self.free = list(range(self.num_slots))
        self.owner = [None] * self.num_slots


class RecurrentStatePool:
    """Device tensors for every layer's recurrent state."""

    def __init__(self, layer_shapes: Sequence[Sequence[Tuple[int, ...]]],
                 num_slots: int, device):
        self.num_slots = num_slots
        self.device = torch.device(device)
        self._layers: List[List[torch.Tensor]] = [
            [torch.zeros((num_slots,) + tuple(shape), dtype=torch.float32,
                         device=self.device) for shape in shapes]
            for shapes in layer_shapes]
        self.nbytes = sum(t.numel() * 4 for ts in self._layers for t in ts)

    def layer(self, i: int) -> List[torch.Tensor]:
        return self._layers[i]

    @property
    def has_state(self) -> bool:
        return any(self._layers)
