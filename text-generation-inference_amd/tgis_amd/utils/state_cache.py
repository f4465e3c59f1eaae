"""Recurrent state slots: the counterpart of the paged KV cache for layers whose memory of a sequence has a fixed size.

A slot holds, for every recurrent layer of the model, two fp32 tensors whose shapes the layer's mixer names: its matrix
state (per head, key channel x value channel) and what it remembers of the last inputs — the last token's mixer input of
RWKV-style token shift ([width]), or the last taps - 1 inputs of a short convolution ([taps - 1, channels]).  A request owns
one slot from its first token to its last; membership changes move slot ids, never state bytes.  Slots are NOT cleared when
they change hands: the kernels start a sequence from zeros whenever its step begins at position 0 (csrc/wkv.hip,
csrc/delta_rule.hip), so a stale slot cannot leak into a new request.

One slot more than `num_slots` is allocated: the NULL slot (id num_slots), never handed out — the inactive rows of a padded
decode graph read and write it, like the null page of the KV pool."""
import heapq
from typing import List, Optional, Sequence, Tuple

import torch


class OutOfSlots(RuntimeError):
    """No free state slot: maps to RESOURCE_EXHAUSTED like OutOfPages."""


class RecurrentStateCache:
    def __init__(self, layer_shapes: Sequence[Optional[Tuple[int, int]]], width: int, num_slots: int, device):
        """layer_shapes[i] describes layer i's recurrence, None for layers without one:
          (heads, head width)                     square matrix state [H, d, d] and a shift row [width] (token-shift mixers);
          {"matrix": shape, "memory": shape}      any per-slot shapes (a delta rule with a convolution tail, ...)."""
        self.num_slots = num_slots
        self.null_slot = num_slots
        self.width = width

        def shapes(s):
            if isinstance(s, dict):
                return tuple(s["matrix"]), tuple(s["memory"])
            return (s[0], s[1], s[1]), (width,)

        self.state = [None if s is None else torch.zeros((num_slots + 1, *shapes(s)[0]), dtype=torch.float32, device=device)
                      for s in layer_shapes]
        self.shift = [None if s is None else torch.zeros((num_slots + 1, *shapes(s)[1]), dtype=torch.float32, device=device)
                      for s in layer_shapes]
        self._free = list(range(num_slots))

    @property
    def free_slots(self) -> int:
        return len(self._free)

    def bytes_per_slot(self) -> int:
        return sum(4 * (s[0].numel() + m[0].numel()) for s, m in zip(self.state, self.shift) if s is not None)

    def alloc(self, n: int) -> List[int]:
        """The n lowest free slot ids.  All or nothing."""
        if n > len(self._free):
            raise OutOfSlots(f"state slots exhausted: need {n}, {len(self._free)} free of {self.num_slots}")
        return [heapq.heappop(self._free) for _ in range(n)]

    def free(self, slots: List[int]):
        for s in slots:
            heapq.heappush(self._free, s)
