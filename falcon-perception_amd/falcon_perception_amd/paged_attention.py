"""Paged KV cache with the reference's interface, backed by gfx950 kernels.

Mirrors `falcon_perception/paged_attention.py:27-393` of the reference: same
constructor, attributes and methods, so the reference's engine
(`paged_inference.py`, `paged_ocr_inference.py`) can drive it unchanged.  The
allocator is host-side integer bookkeeping as in the reference; every device
operation on K/V data (append, block-id lookup) is a HIP kernel reached through
`ops`, and the masks it hands out are consumed by the kernels in `attention.py`.
"""

from __future__ import annotations

from typing import NamedTuple

import torch
from torch import Tensor
from torch.nn.attention.flex_attention import BlockMask, noop_mask

from . import ops
from .attention import HybridPrefillMask, PagedDecodeMask, get_causal_mask_mod
from .kv_cache import KVCacheBase


def _cdiv(x, multiple) -> int:
    return int((x + multiple - 1) // multiple)


class StepMeta(NamedTuple):
    """What `insert_kv` saw last: the attention call of the same layer reads it."""

    layer_id: int
    input_pos: Tensor
    batch_idx: Tensor


class PagedKVCache(KVCacheBase):
    """Page pool, page table and allocator of the paged engine (`paged_attention.py:27-393`).

    State (all public, as in the reference):
      kv_cache            [L, 2, 1, H, n_pages * page_size, D] zeros; a page is
                          page_size * D contiguous elements per head (:72-74)
      page_table          [max_batch, n_pages] int64, -1 = unmapped; row 0 is all 0 (:58-59)
      physical_to_logical [max_batch, n_pages] int64 inverse map (:70)
      page_table_cpu, capacity, free_pages, free_batch_idx   host mirrors (:60-67);
                          page 0 and batch slot 0 are reserved and never handed out

    `max_blocks_per_seq` (not an argument of the reference's class) makes the tables sparse:
    page_table becomes [max_batch, max_blocks_per_seq] and the inverse table is not kept.  The
    reference's dense [max_batch, n_pages] int64 pair grows with pool size times batch size
    (1.4 GB for 257 slots over a 343 k-page pool); the kernels only ever read
    page_table[slot, block], so the narrow table serves them unchanged.  What needs the inverse
    table (`get_mask_mod`, the element mask of the reference's flex kernels) is then unavailable.
    """

    default_kv_rep = 1  # kv_rep of caches created from now on, see `falcon_perception_amd.install`
    default_qk_normalised = False  # likewise: whether the q and k rows the model produces have norm sqrt(head_dim)

    def __init__(self, n_pages: int, page_size: int, max_batch_size: int, n_heads: int, head_dim: int,
                 num_layers: int, dtype: torch.dtype, device: str | torch.device = "cuda",
                 max_blocks_per_seq: int | None = None):
        self.n_pages = n_pages
        self.page_size = page_size
        self.max_batch_size = max_batch_size
        self.dtype = dtype
        self.device = device

        self.table_cols = n_pages if max_blocks_per_seq is None else int(max_blocks_per_seq)
        if not 0 < self.table_cols <= n_pages:
            raise ValueError("max_blocks_per_seq must be between 1 and n_pages")
        self.page_table = torch.full((max_batch_size, self.table_cols), -1, dtype=torch.int64, device=device)
        self.page_table[0].zero_()
        self.physical_to_logical = None
        if max_blocks_per_seq is None:
            self.physical_to_logical = torch.full((max_batch_size, n_pages), -1, dtype=torch.int64, device=device)
        self.page_table_cpu: list[list[int]] = [[] for _ in range(max_batch_size)]
        self.capacity: list[int] = [0] * max_batch_size
        self.free_pages: list[int] = list(range(n_pages - 1, 0, -1))
        self.free_batch_idx: list[int] = list(range(max_batch_size - 1, 0, -1))

        self.kv_shape = (num_layers, 2, 1, n_heads, n_pages * page_size, head_dim)
        self.kv_cache = torch.zeros(self.kv_shape, dtype=dtype, device=device)
        # views of every layer's K and V planes, made once: [H, N, D] for the kernels, [1, H, N, D] as returned
        # to the model (an indexing operation per layer and call costs the host more than the launch itself)
        self._planes = [(self.kv_cache[l, 0, 0], self.kv_cache[l, 1, 0]) for l in range(num_layers)]
        self._pools = [(self.kv_cache[l, 0], self.kv_cache[l, 1]) for l in range(num_layers)]

        # 1, or n_heads // n_kv_heads when the cached V heads are plain copies inside a group (the model's
        # repeat_kv, model.py:112-113): the decode kernel then reads V once per group.  Taken from the class
        # default (`falcon_perception_amd.install(kv_rep=...)` sets it for an engine that is not edited) when
        # it divides this cache's head count.
        self.kv_rep = self.default_kv_rep if n_heads % self.default_kv_rep == 0 else 1
        # Whether every q and k row has norm sqrt(head_dim): the reference's model RMS-normalises both without a
        # weight and rotates them (model.py:110-116).  |scale * q.k| is then at most scale * head_dim, and the
        # bf16 prefill kernel runs its softmax without a running maximum (`score_bound`).  Set by
        # `insert_qkv_norm_rope`, which does the normalisation itself, or by `install(qk_norm=True)`.
        self.qk_normalised = self.default_qk_normalised

        # what the attention callables need from the step in flight
        self.last_decode_step: StepMeta | None = None
        self.last_prefill_step: StepMeta | None = None
        self._workspace: Tensor | None = None
        self._decode_launch: dict[tuple, tuple[int, int]] = {}
        self._prefill_workspace: Tensor | None = None
        self._prefill_need: dict[tuple, int] = {}

    # ------------------------------------------------------------------ append
    def insert_kv(self, layer_id: int, k: Tensor, v: Tensor, input_pos: Tensor | None = None,
                  batch_idx: Tensor | None = None, **kwargs):
        """Append k, v; 1-D batch_idx = decode, 2-D [1, L] = packed prefill (:76-93)."""
        del kwargs
        assert input_pos is not None, "input_pos is required for paged kv cache"
        assert batch_idx is not None, "batch_idx is required for paged kv cache"
        assert batch_idx.ndim in [1, 2], "batch_idx must be 1D (decode) or 2D (prefill 1xL)"
        if batch_idx.ndim == 1:
            return self.assign(layer_id, batch_idx, input_pos, k, v)
        return self.assign_prefill_no_paging(layer_id, k, v, input_pos, batch_idx)

    def assign(self, layer_id: int, batch_idx: Tensor, input_pos: Tensor, k_val: Tensor, v_val: Tensor):
        """Decode append (:184-232): k_val, v_val [B, H, S, D] go to the slots of
        (batch_idx[b], input_pos[b, s]); unmapped (-1) pages are redirected to the
        reserved page 0.  Returns the layer's whole K and V pools, [1, H, N, D] views."""
        B, H, S, K_D = k_val.shape
        _, _, _, H_cache, MAX_S, D_cache = self.kv_cache.shape
        assert H_cache == H, "number of heads must match"
        assert MAX_S >= S, "cache must have enough space"
        assert D_cache == K_D, "hidden dim must match"
        assert input_pos.shape == (B, S), "input_pos must have the same shape as val"
        assert batch_idx.shape == (B,), "batch_idx must have one dimension only"
        pool_k, pool_v = self._planes[layer_id]
        ops.kv_append(pool_k, pool_v, k_val, v_val, self.page_table, batch_idx, input_pos, self.page_size,
                      clamp_negative=True)
        self.last_decode_step = StepMeta(layer_id, input_pos, batch_idx)
        return self._pools[layer_id]

    def assign_prefill_no_paging(self, layer_id: int, k_val: Tensor, v_val: Tensor, input_pos: Tensor,
                                 batch_idx: Tensor):
        """Prefill append (:364-393): k_val, v_val [1, H, L, D], input_pos, batch_idx [1, L].
        Padding rows carry (batch_idx 0, pos 0) and land in slot 0 of the reserved page.
        Returns the inputs, as the reference does."""
        assert batch_idx.ndim == 2, "batch_idx must be a 2D tensor"
        assert batch_idx.shape[0] == 1, "batch_idx must have batch size 1"
        assert input_pos.ndim == 2, "input_pos must be a 2D tensor"
        assert k_val.ndim == 4, "k_val must be a 4D tensor"
        assert v_val.ndim == 4, "v_val must be a 4D tensor"
        pool_k, pool_v = self._planes[layer_id]
        # [1, H, L, D] seen as L row groups of one token each: the strides say so, no views are made
        ops.kv_append(pool_k, pool_v, k_val, v_val, self.page_table, batch_idx, input_pos, self.page_size,
                      clamp_negative=False, packed=True)
        self.last_prefill_step = StepMeta(layer_id, input_pos, batch_idx)
        return k_val, v_val

    def insert_qkv_norm_rope(self, layer_id: int, xq: Tensor, xk: Tensor, xv: Tensor, freqs_cis: Tensor,
                             freqs_cis_2d: Tensor | None = None, *, input_pos: Tensor, batch_idx: Tensor):
        """`Attention._pre_attention` from the QK norm on (`model.py:110-119`) and `insert_kv`
        (`model.py:150-153`) in one launch; not a method of the reference's class.

        xq [B, S, n_heads, D], xk / xv [B, S, n_kv_heads, D]: the reshaped slices of the qkv
        projection (`model.py:106-109`), views are fine.  Returns (q [B, n_heads, S, D], K, V) where
        K, V are what `insert_kv` returns for a decode step (the layer's pool views); a prefill step
        gets the pool views as well instead of the rotated fresh rows, which the paged prefill
        attention does not read."""
        decode = batch_idx.ndim == 1
        assert batch_idx.ndim in [1, 2], "batch_idx must be 1D (decode) or 2D (prefill 1xL)"
        B, S = xq.shape[0], xq.shape[1]
        assert input_pos.shape == (B, S), "input_pos must be [B, S]"
        if decode:
            assert S == 1 and batch_idx.shape == (B,), "a decode step has one token per sequence"
        else:
            assert B == 1 and batch_idx.shape == (1, S), "a prefill step is one packed row"
        q = ops.qkv_norm_rope_append(xq, xk, xv, freqs_cis, freqs_cis_2d, *self._planes[layer_id], self.page_table,
                                     batch_idx, input_pos, self.page_size, clamp_negative=decode)
        self.qk_normalised = True  # every row this call wrote or returned has norm sqrt(head_dim)
        if decode:
            self.last_decode_step = StepMeta(layer_id, input_pos, batch_idx)
        else:
            self.last_prefill_step = StepMeta(layer_id, input_pos, batch_idx)
        return (q, *self._pools[layer_id])

    def v_copies_are_identical(self, layer_id: int = 0) -> bool:
        """Whether the V plane of a layer really holds `kv_rep` identical heads per group (bit for bit, over
        the whole pool): the condition under which decoding with `kv_rep` > 1 equals the plain read.  A check
        for bring-up; it reads the plane and waits for the result."""
        if self.kv_rep == 1:
            return True
        v = self.kv_cache[layer_id, 1, 0]
        groups = v.view(v.shape[0] // self.kv_rep, self.kv_rep, *v.shape[1:])
        bits = groups.view(torch.int16 if v.element_size() == 2 else torch.int32)
        return bool((bits == bits[:, :1]).all())

    # --------------------------------------------------------------- allocator
    @property
    def num_free_pages(self) -> int:
        return len(self.free_pages)

    def can_reserve(self, size: int, batch_idx_int: int | None = None) -> bool:
        """Host-only admission check (:95-100)."""
        if batch_idx_int is None:
            return self.num_free_pages * self.page_size >= size and len(self.free_batch_idx) > 0
        return self.reserve(batch_idx_int, None, size, dry_run=True)

    def allocate(self) -> int:
        """Take a free batch slot and clear its table rows (:102-109)."""
        slot = self.free_batch_idx.pop()
        self.capacity[slot] = 0
        if self.physical_to_logical is not None:
            self.physical_to_logical[slot].fill_(-1)
        self.page_table[slot].fill_(-1)
        return slot

    def reserve(self, batch_idx_int: int, batch_idx: Tensor | None, seq_len: int, dry_run: bool = False) -> bool:
        """Grow slot `batch_idx_int` to hold `seq_len` tokens (:115-164).

        New pages are the tail of `free_pages` in list order; they are mapped to the
        next logical blocks of the slot.  Raises RuntimeError when the pool is short
        (`dry_run=True` returns the answer instead)."""
        have = self.capacity[batch_idx_int]
        if seq_len <= have:
            return True
        n_new = _cdiv(seq_len - have, self.page_size)
        fits = bool(n_new <= self.num_free_pages)
        if have // self.page_size + n_new > self.table_cols:  # only a sparse table can be narrower than the pool
            if dry_run:
                return False
            raise RuntimeError(
                f"Cannot reserve a sequence of length {seq_len} in batch {batch_idx_int}: "
                f"the page table holds {self.table_cols} blocks of {self.page_size} tokens per sequence."
            )
        if dry_run:
            return fits
        if not fits:
            raise RuntimeError(
                f"Cannot reserve {n_new} pages for a sequence of length {seq_len} "
                f"in batch {batch_idx_int}. Only {self.num_free_pages} pages available. "
                f"Current capacity is {have} tokens."
            )
        first = have // self.page_size
        pages = self.free_pages[-n_new:]
        del self.free_pages[-n_new:]
        pages_dev = torch.tensor(pages, device=self.device)
        row = batch_idx_int  # the tensor argument of the reference names the same slot
        self.page_table[row, first:first + n_new] = pages_dev
        if self.physical_to_logical is not None:
            self.physical_to_logical[row, pages_dev] = torch.arange(first, first + n_new, device=self.device)
        self.page_table_cpu[batch_idx_int] += pages
        self.capacity[batch_idx_int] = have + n_new * self.page_size
        return True

    def erase(self, batch_idx: int) -> None:
        """Release a slot and its pages; table rows go back to -1, pool bytes stay (:166-182)."""
        self.free_batch_idx.append(batch_idx)
        self.free_pages.extend(reversed(self.page_table_cpu[batch_idx]))
        self.page_table_cpu[batch_idx] = []
        self.page_table[batch_idx].fill_(-1)
        if self.physical_to_logical is not None:
            self.physical_to_logical[batch_idx].fill_(-1)
        self.capacity[batch_idx] = 0

    # ------------------------------------------------------------------- masks
    def convert_logical_block_mask(self, block_mask: BlockMask, batch_idx: Tensor | None = None) -> PagedDecodeMask:
        """Logical block mask -> mask over physical pages (:234-301).

        The returned object is what `compiled_flex_attn_decode` consumes; its
        `kv_indices` / `full_kv_indices` (physical page ids, zero tail of width
        n_pages) are produced by the block-id kernel when somebody reads them."""
        B = block_mask.kv_indices.shape[0]
        if block_mask.BLOCK_SIZE[1] != self.page_size:
            raise RuntimeError(
                f"Expect block_mask has the same column block size as page_size"
                f"but got size={block_mask.BLOCK_SIZE[1]} and size={self.page_size}"
            )
        if batch_idx is None:
            batch_idx = torch.arange(B, device=block_mask.kv_num_blocks.device)
        assert batch_idx.ndim == 1, "batch_idx must be a 1D tensor"
        assert batch_idx.shape[0] == B, "batch_idx must have the same shape as block_mask"
        assert B <= self.max_batch_size, "batch_idx must be less than or equal to max_batch_size"
        return PagedDecodeMask(self, block_mask, batch_idx)

    def get_logical_kv_idx(self, physical_batch_idx: Tensor, physical_kv_idx: Tensor, batch_idx: Tensor):
        """Physical slot -> (mapped?, logical position) for one batch row (:303-311)."""
        if self.physical_to_logical is None:
            raise RuntimeError("this cache was built with max_blocks_per_seq: it keeps no physical_to_logical table")
        slot_row = batch_idx[physical_batch_idx]
        block = self.physical_to_logical[slot_row, physical_kv_idx // self.page_size]
        logical = block * self.page_size + physical_kv_idx % self.page_size
        return block >= 0, logical.clamp(min=0)

    def get_mask_mod(self, mask_mod, batch_idx: Tensor):
        """mask_mod over physical slots: unmapped slots are masked, mapped ones defer
        to the logical `mask_mod` (:313-333)."""
        inner = noop_mask if mask_mod is None else mask_mod

        def physical_mask_mod(b, h, q_idx, physical_kv_idx):
            mapped, logical = self.get_logical_kv_idx(b, physical_kv_idx, batch_idx)
            return torch.where(mapped, inner(b, h, q_idx, logical), False)

        return physical_mask_mod

    def create_causal_blockmask(self, B: int, L: int) -> BlockMask:
        """Causal BlockMask [B, 1, L/P, L/P] with block size = page size (:335-341).

        Built in closed form instead of evaluating the mask on a dense grid: query
        block i has the partial block {i} and the full blocks 0..i-1; index rows list
        present blocks first, then the rest ascending, as torch's create_block_mask does."""
        P = self.page_size
        n = _cdiv(L, P)
        dev = self.device
        ar = torch.arange(n, dtype=torch.int32, device=dev)
        # row i of the partial list: [i, 0, 1, .., i-1, i+1, ..]
        col = ar.view(1, n).expand(n, n)
        row = ar.view(n, 1)
        partial_idx = torch.where(col == 0, row, torch.where(col <= row, col - 1, col))
        full_idx = col.contiguous()
        kv_num = torch.ones(n, dtype=torch.int32, device=dev)
        full_num = ar.clone()
        # a ragged last block (L % P != 0) stays partial in every row that reaches it
        expand = lambda t: t.view(1, 1, *t.shape).expand(B, 1, *t.shape).contiguous()
        return BlockMask.from_kv_blocks(
            expand(kv_num), expand(partial_idx.contiguous()), expand(full_num), expand(full_idx),
            BLOCK_SIZE=(P, P), mask_mod=get_causal_mask_mod(), seq_lengths=(L, L),
        )

    def create_prefill_blockmask(self, batch_idx: Tensor, input_ids: Tensor, soi_id: int, eoi_id: int,
                                 BLOCK_SIZE: int = 128, *, open_spans=None, validate: bool = True) -> HybridPrefillMask:
        """Mask of a packed prefill step: document-causal OR image-prefix (:343-362).

        `open_spans` and `validate` are not arguments of the reference: `open_spans` lists the cache slots
        whose chunk begins inside an image span that an earlier chunk opened; with `validate` (default) a
        packed row whose spans cross a document boundary, the end of the row, or start before it undeclared
        raises RuntimeError (one host read of a device word) instead of yielding a wrong mask."""
        assert batch_idx.ndim == 2 and batch_idx.shape[0] == 1
        return HybridPrefillMask(self, batch_idx, input_ids, soi_id, eoi_id, BLOCK_SIZE,
                                 open_spans=open_spans, validate=validate)

    # ------------------------------------------------ decode launch parameters
    def decode_split_tokens(self, B: int, Hc: int, max_context: int) -> int:
        return ops.decode_split_tokens(B, Hc, max_context, self.page_size)

    def decode_workspace(self, B: int, Hq: int, D: int, max_context: int, Hc: int) -> Tensor | None:
        """Split-K scratch of the decode kernel, owned by the cache.

        Sized on first use for the largest batch and the finest split any batch size
        can get, so its address never changes afterwards: HIP graphs captured for
        one batch bucket stay valid when another bucket runs."""
        return self.decode_launch(B, Hq, D, max_context, Hc)[0]

    def decode_launch(self, B: int, Hq: int, D: int, max_context: int, Hc: int) -> tuple[Tensor | None, int]:
        """(workspace, split_tokens) of a decode launch of this shape.  The library is asked once per shape;
        every later layer and step of the same batch bucket takes the answer from a dictionary, so an eager
        decode step crosses into the library once per layer, for the launch itself."""
        key = (B, Hq, D, max_context, Hc)
        hit = self._decode_launch.get(key)
        if hit is None:
            worst_b = max(B, self.max_batch_size)
            finest = min(self.decode_split_tokens(1, Hc, max_context),
                         self.decode_split_tokens(worst_b, Hc, max_context))
            need = ops.decode_workspace_bytes(worst_b, Hq, D, max_context, finest)
            if need and (self._workspace is None or self._workspace.numel() < need):
                self._workspace = torch.empty(need, dtype=torch.uint8, device=self.kv_cache.device)
            hit = (need, self.decode_split_tokens(B, Hc, max_context))
            self._decode_launch[key] = hit
        return (self._workspace if hit[0] else None), hit[1]

    def score_bound(self, head_dim: int, scale: float | None) -> float:
        """Bound of |scale * q.k| the prefill kernel may rely on: 0 (unknown) unless q and k are normalised;
        then scale * head_dim with a tenth of slack for the roundings after the norm and the rotation."""
        if not self.qk_normalised:
            return 0.0
        return 1.1 * head_dim * (head_dim ** -0.5 if scale is None else abs(scale))

    def prefill_workspace(self, Lq: int, Hq: int, D: int, Hc: int, dtype: torch.dtype):
        """Scratch with which the prefill kernel cuts a small launch along the keys as well, owned by the
        cache and grown on demand (prefill steps are not captured in graphs); False when the shape needs none."""
        key = (Lq, Hq, Hc, D, dtype)
        need = self._prefill_need.get(key)
        if need is None:
            need = self._prefill_need[key] = ops.prefill_workspace_bytes(Lq, Hq, Hc, D, dtype)
        if need == 0:
            return False
        if self._prefill_workspace is None or self._prefill_workspace.numel() < need:
            self._prefill_workspace = torch.empty(need, dtype=torch.uint8, device=self.kv_cache.device)
        return self._prefill_workspace
