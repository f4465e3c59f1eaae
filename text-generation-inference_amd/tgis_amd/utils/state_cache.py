"""Recurrent state slots: the counterpart of the paged KV cache for layers whose memory of a sequence has a fixed size.

A slot holds, for every recurrent layer of the model, the fp32 matrix state of each head ([H, d, d]: key channel x value
channel) and the fp32 input of the sequence's last token (the "token shift" of RWKV-style mixers).  A request owns one slot
from its first token to its last; membership changes move slot ids, never state bytes.  Slots are NOT cleared when they
change hands: the kernels start a sequence from zeros whenever its step begins at position 0 (csrc/wkv.hip), so a stale
slot cannot leak into a new request.

One slot more than `num_slots` is allocated: the NULL slot (id num_slots), never handed out — the inactive rows of a padded
decode graph read and write it, like the null page of the KV pool."""
import heapq
from typing import List, Optional, Sequence, Tuple

import torch


class OutOfSlots(RuntimeError):
    """No free state slot: maps to RESOURCE_EXHAUSTED like OutOfPages."""


class RecurrentStateCache:
    def __init__(self, layer_shapes: Sequence[Optional[Tuple[int, int]]], width: int, num_slots: int, device):
        """layer_shapes[i] = (heads, head width) of layer i's recurrence, or None for layers without one."""
        self.num_slots = num_slots
        self.null_slot = num_slots
        self.width = width
        self.state = [None if s is None else torch.zeros((num_slots + 1, s[0], s[1], s[1]), dtype=torch.float32, device=device)
                      for s in layer_shapes]
        self.shift = [None if s is None else torch.zeros((num_slots + 1, width), dtype=torch.float32, device=device)
                      for s in layer_shapes]
        self._free = list(range(num_slots))

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def bytes_per_slot(self) -> int:
        return sum(4 * (s[0].numel() + self.width) for s in self.state if s is not None)

    def alloc(self, n: int) -> List[int]:
        """The n lowest free slot ids.  All or nothing."""
        if n > len(self._free):
            raise OutOfSlots(f"state slots exhausted: need {n}, {len(self._free)} free of {self.num_slots}")
        return [heapq.heappop(self._free) for _ in range(n)]

    def free(self, slots: List[int]):
        for s in slots:
            heapq.heappush(self._free, s)
