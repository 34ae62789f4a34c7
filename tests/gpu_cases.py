"""Seeded paged-cache states for the GPU parity tests.

Values are drawn on the CPU with a seeded torch.Generator and then cast and moved,
so the oracle and the HIP path see bit-identical inputs on any machine.
"""

from __future__ import annotations

import numpy as np
import torch

from falcon_perception_amd.paged_attention import PagedKVCache
from oracle import paged_kv_oracle as O

DEV = "cuda"


def bits(t: torch.Tensor) -> np.ndarray:
    """Raw bit pattern of a tensor as a numpy integer array (bf16 has no numpy dtype)."""
    t = t.detach().contiguous().cpu()
    view = {4: torch.int32, 2: torch.int16, 8: torch.int64}[t.element_size()]
    return t.view(view).numpy()


def f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def randn(gen, shape, dtype):
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype)


class PagedState:
    """A PagedKVCache on the GPU plus an oracle mirror of its tables and pool."""

    def __init__(self, seed, *, n_pages, page_size, max_batch, Hc, D, dtype, n_layers=1, shuffle=True,
                 max_blocks_per_seq=None):
        self.gen = torch.Generator().manual_seed(seed)
        self.cache = PagedKVCache(n_pages, page_size, max_batch, Hc, D, n_layers, dtype, device=DEV,
                                  max_blocks_per_seq=max_blocks_per_seq)
        self.mirror = O.PagedAllocator(n_pages, page_size, max_batch)
        if shuffle:
            perm = (torch.randperm(n_pages - 1, generator=self.gen) + 1).tolist()
            self.cache.free_pages = list(perm)
            self.mirror.free_pages = list(perm)
        self.dtype = dtype
        self.P = page_size
        self.Hc, self.D = Hc, D
        self.slots: list[int] = []
        self.lens: list[int] = []

    def add_sequence(self, length: int) -> int:
        b = self.cache.allocate()
        assert b == self.mirror.allocate()
        self.cache.reserve(b, torch.tensor([b], device=DEV), length)
        self.mirror.reserve(b, length)
        self.slots.append(b)
        self.lens.append(length)
        return b

    def prefill_random(self, layer=0, pad_to=1):
        """Fill every sequence with N(0,1) K/V through the packed prefill append."""
        bidx, pos = [], []
        for b, L in zip(self.slots, self.lens):
            gap = (-L) % pad_to
            bidx += [b] * L + [0] * gap
            pos += list(range(L)) + [0] * gap
        Lp = len(bidx)
        k = randn(self.gen, (1, self.Hc, Lp, self.D), self.dtype)
        v = randn(self.gen, (1, self.Hc, Lp, self.D), self.dtype)
        bt = torch.tensor([bidx], dtype=torch.int64)
        pt = torch.tensor([pos], dtype=torch.int64)
        rk, rv = self.cache.insert_kv(layer, k.to(DEV), v.to(DEV), input_pos=pt.to(DEV), batch_idx=bt.to(DEV))
        return k, v, bt, pt, rk, rv

    def pool_planes(self, layer=0):
        return self.cache.kv_cache[layer, 0, 0], self.cache.kv_cache[layer, 1, 0]


def check_tables_match(state: PagedState):
    assert state.cache.page_table.cpu().numpy().tolist() == state.mirror.page_table.tolist()
    assert state.cache.physical_to_logical.cpu().numpy().tolist() == state.mirror.physical_to_logical.tolist()
