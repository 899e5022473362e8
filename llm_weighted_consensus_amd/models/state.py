"""Recurrent-state slots for decoders whose layers carry per-sequence state besides keys and values (a running
matrix of a linear-attention layer, the last inputs of a causal convolution).

One fp32 pool ``[num_slots + 1, slot_elems]`` holds, per slot, every field of every layer; a field is the strided
view ``[num_slots + 1, *shape]``.  Slot ids come from the engine's C++ block manager (``set_state_slots``): a
sequence holds one slot from admission to its end, forks copy a slot, preemption saves and restores it.  The last
slot (``scratch``) belongs to no sequence: padded rows of a decode bucket and warm-up runs write there.

Kernels never read a slot for positions before a sequence's start, so slots are handed out again without clearing.
"""
from __future__ import annotations

import math
from typing import Dict, List, Sequence, Tuple

import torch


class RecurrentStatePool:
    def __init__(self, fields: Sequence[Tuple[str, Tuple[int, ...]]], num_slots: int, device):
        """``fields``: (name, shape) per state tensor of one sequence."""
        self.num_slots = int(num_slots)
        self.scratch = self.num_slots
        offs, o = [], 0
        for _name, shape in fields:
            offs.append(o)
            o += -(-max(1, math.prod(shape)) // 4) * 4  # every view starts on a 16-byte boundary
        self.slot_elems = max(o, 4)
        self.pool = torch.zeros(self.num_slots + 1, self.slot_elems, dtype=torch.float32, device=device)
        self.fields: Dict[str, torch.Tensor] = {}
        for (name, shape), off in zip(fields, offs):
            n = math.prod(shape)
            self.fields[name] = self.pool[:, off:off + n].view(self.num_slots + 1, *shape)

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.fields[name]

    @staticmethod
    def bytes_per_slot(fields: Sequence[Tuple[str, Tuple[int, ...]]]) -> int:
        return 4 * sum(-(-max(1, math.prod(s)) // 4) * 4 for _n, s in fields)

    def copy_slots(self, pairs) -> None:
        """(src, dst) slot copies queued by the block manager's forks."""
        pairs = list(pairs)
        if pairs:
            p = torch.tensor(pairs, dtype=torch.int64, device=self.pool.device).view(-1, 2)
            self.pool.index_copy_(0, p[:, 1], self.pool.index_select(0, p[:, 0]))

    def take(self, slots: List[int]) -> torch.Tensor:
        """The contents of ``slots``: [n, slot_elems] (preemption: saved beside the swapped-out blocks)."""
        return self.pool.index_select(0, torch.tensor(list(slots), dtype=torch.int64, device=self.pool.device))

    def put(self, slots: List[int], data: torch.Tensor) -> None:
        self.pool.index_copy_(0, torch.tensor(list(slots), dtype=torch.int64, device=self.pool.device),
                              data.to(self.pool.device))
