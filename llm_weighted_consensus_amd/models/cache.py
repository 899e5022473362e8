"""Paged K/V cache for decoders whose layers differ (key size != value size, other head counts per layer).

One pool ``[num_blocks, block_elems]`` holds, per block, every layer's keys then values for ``block_size`` tokens;
a layer's K is the strided view ``[num_blocks, block_size, G*D]`` (token-major rows) and its V the 4-token
interleaved view ``[num_blocks, block_size/4, G*Dv, 4]`` — four consecutive tokens of one value column are one
8-byte word, the matrix cores' operand for the weighted sum without a transpose (``csrc/kernels/res32/wattn.hip``).  Block ids come from the engine's C++ block
manager like every other model's; whole blocks are copied (copy-on-write forks), exported and imported (swap,
prefill hand-over) with one index operation on the pool."""
from __future__ import annotations

from typing import List, Sequence, Tuple

import torch


class PagedLayerCache:
    def __init__(self, layer_dims: Sequence[Tuple[int, int]], num_blocks: int, block_size: int, device,
                 dtype=torch.bfloat16):
        """``layer_dims``: per layer (G*D, G*Dv), the key and value row sizes."""
        self.num_blocks, self.block_size, self.dtype = int(num_blocks), int(block_size), dtype
        if block_size % 4:
            raise ValueError("PagedLayerCache: block_size must be a multiple of 4 (4-token interleaved values)")
        self.layer_dims = [(int(a), int(b)) for a, b in layer_dims]
        offs, o = [], 0
        for nk, nv in self.layer_dims:
            ko = o
            o += -(-block_size * nk // 8) * 8  # every view starts on a 16-byte boundary
            vo = o
            o += -(-block_size * nv // 8) * 8
            offs.append((ko, vo))
        self.block_elems = o
        self.pool = torch.zeros(self.num_blocks, self.block_elems, dtype=dtype, device=device)
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        for (nk, nv), (ko, vo) in zip(self.layer_dims, offs):
            self.k.append(self.pool[:, ko:ko + block_size * nk].view(self.num_blocks, block_size, nk))
            self.v.append(self.pool[:, vo:vo + block_size * nv].view(self.num_blocks, block_size // 4, nv, 4))

    @staticmethod
    def elems_per_block(layer_dims: Sequence[Tuple[int, int]], block_size: int) -> int:
        return sum(-(-block_size * nk // 8) * 8 + -(-block_size * nv // 8) * 8 for nk, nv in layer_dims)

    # token rows by cache slot (slot = block * block_size + offset): tools and tests, not the product path
    def rows(self, layer: int, slots: torch.Tensor):
        """(K rows [n, G*D], V rows [n, G*Dv]) of the tokens at ``slots`` (int64)."""
        b, o = slots // self.block_size, slots % self.block_size
        return self.k[layer][b, o], self.v[layer][b, o // 4, :, o % 4]

    def set_rows(self, layer: int, slots: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> None:
        b, o = slots // self.block_size, slots % self.block_size
        self.k[layer][b, o] = k.to(self.pool.dtype)
        self.v[layer][b, o // 4, :, o % 4] = v.to(self.pool.dtype)

    def copy_blocks(self, pairs: torch.Tensor) -> None:
        """(src, dst) block copies queued by the block manager's copy-on-write."""
        if pairs.numel():
            p = pairs.view(-1, 2).long()
            self.pool.index_copy_(0, p[:, 1], self.pool.index_select(0, p[:, 0]))

    def take_blocks(self, idx: torch.Tensor) -> torch.Tensor:
        """The contents of blocks ``idx`` (int64), every layer: [n, block_elems]."""
        return self.pool.index_select(0, idx)

    def put_blocks(self, idx: torch.Tensor, data: torch.Tensor) -> None:
        self.pool.index_copy_(0, idx, data.to(self.pool.device))

    @staticmethod
    def num_exported(data: torch.Tensor) -> int:
        return int(data.shape[0]) if data.dim() == 2 else 0
