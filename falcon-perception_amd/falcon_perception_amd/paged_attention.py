"""Paged KV cache with the reference's interface, backed by gfx950 kernels.

Mirrors `falcon_perception/paged_attention.py:27-393` of the reference: same
constructor, attributes and methods, so the reference's engine
(`paged_inference.py`, `paged_ocr_inference.py`) can drive it unchanged.  The
allocator is host-side integer bookkeeping as in the reference; every device
operation on K/V data (append, block-id lookup) is a HIP kernel reached through
`ops`, and the masks it hands out are consumed by the kernels in `attention.py`.
"""

from __future__ import annotations

import warnings
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
    """What `insert_kv` saw last: the attention call of the same layer reads it.  `k_new` / `v_new` are the
    rows of a decode step whose append has been left to the attention launch (`fuse_decode_append`)."""

    layer_id: int
    input_pos: Tensor
    batch_idx: Tensor
    k_new: Tensor | None = None
    v_new: Tensor | None = None


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

    # what `falcon_perception_amd.install` sets for the caches an unedited engine creates afterwards
    default_kv_rep = 1
    default_qk_normalised = False
    default_fuse_decode_append = False

    def __init__(self, n_pages: int, page_size: int, max_batch_size: int, n_heads: int, head_dim: int,
                 num_layers: int, dtype: torch.dtype, device: str | torch.device = "cuda",
                 max_blocks_per_seq: int | None = None, *, kv_rep: int | None = None,
                 qk_normalised: bool | None = None, fuse_decode_append: bool | None = None):
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
        self._kv = torch.zeros(self.kv_shape, dtype=dtype, device=device)  # `kv_cache`, see the property
        # views of every layer's K and V planes, made once: [H, N, D] for the kernels, [1, H, N, D] as returned
        # to the model (an indexing operation per layer and call costs the host more than the launch itself)
        self._planes = [(self._kv[l, 0, 0], self._kv[l, 1, 0]) for l in range(num_layers)]
        self._pools = [(self._kv[l, 0], self._kv[l, 1]) for l in range(num_layers)]

        # 1, or n_heads // n_kv_heads when the cached V heads are plain copies inside a group (the model's
        # repeat_kv, model.py:112-113): the decode kernel then reads V once per group.  An argument of this
        # constructor, or else the class default (`falcon_perception_amd.install(kv_rep=...)` sets it for an
        # engine that is not edited) when it divides this cache's head count.  A value that came from the
        # class default is checked against the V rows of the first prefill step (`_check_v_copies`).
        if kv_rep is None:
            self.kv_rep = self.default_kv_rep if n_heads % self.default_kv_rep == 0 else 1
            self._kv_rep_unverified = self.kv_rep > 1
        else:
            if kv_rep < 1 or n_heads % kv_rep:
                raise ValueError(f"kv_rep={kv_rep} must divide the {n_heads} cached heads")
            self.kv_rep = int(kv_rep)
            self._kv_rep_unverified = False
        # Whether every q and k row has norm sqrt(head_dim): the reference's model RMS-normalises both without a
        # weight and rotates them (model.py:110-116).  |scale * q.k| is then at most scale * head_dim, and the
        # bf16 prefill kernel runs its softmax without a running maximum (`score_bound`).  Set by
        # `insert_qkv_norm_rope`, which does the normalisation itself, or by `install(qk_norm=True)`.
        self.qk_normalised = self.default_qk_normalised if qk_normalised is None else bool(qk_normalised)
        # Whether a decode `insert_kv` leaves its rows to the attention launch of the same layer, which then
        # appends and attends in one kernel (`fp_paged_decode_append`).  The reference's model calls the two
        # back to back (model.py:150-162) and nothing reads the pool in between; whatever else touches the
        # cache first (`flush`, another insert, `kv_cache`, erase, a prefill mask) launches the plain append.
        self.fuse_decode_append = (self.default_fuse_decode_append if fuse_decode_append is None
                                   else bool(fuse_decode_append))

        # what the attention callables need from the step in flight
        self.last_decode_step: StepMeta | None = None
        self.last_prefill_step: StepMeta | None = None
        self._workspace: Tensor | None = None
        self._retired_workspaces: list[Tensor] = []  # graphs captured earlier still write to these
        self._decode_launch: dict[tuple, tuple[int, int]] = {}
        self._decode_plan: Tensor | None = None  # the step's plan of the decode kernel (`decode_plan`)
        self._decode_plan_owner = None           # the mask object it was made for
        self._prefill_workspace: Tensor | None = None
        self._prefill_need: dict[tuple, int] = {}
        self._prefill_tile_rows: dict[tuple, int] = {}
        # status word of the last prefill mask, on its way to the host (`check_prefill_masks`)
        self._mask_status_host: Tensor | None = None
        self._mask_status_event = None

    @property
    def kv_cache(self) -> Tensor:
        """The pool [L, 2, 1, H, n_pages * page_size, D] (`paged_attention.py:73-74`).  Reading it first
        launches an append that is still waiting for its attention call."""
        self.flush()
        return self._kv

    def flush(self) -> None:
        """Launch the append of a decode step whose rows were left to the attention call (no-op otherwise)."""
        step = self.last_decode_step
        if step is None or step.k_new is None:
            return
        self.last_decode_step = step._replace(k_new=None, v_new=None)
        pool_k, pool_v = self._planes[step.layer_id]
        ops.kv_append(pool_k, pool_v, step.k_new, step.v_new, self.page_table, step.batch_idx, step.input_pos,
                      self.page_size, clamp_negative=True)

    # ------------------------------------------------------------------ append
    def insert_kv(self, layer_id: int, k: Tensor, v: Tensor, input_pos: Tensor | None = None,
                  batch_idx: Tensor | None = None, **kwargs):
        """Append k, v; 1-D batch_idx = decode, 2-D [1, L] = packed prefill (:76-93)."""
        del kwargs
        assert input_pos is not None, "input_pos is required for paged kv cache"
        assert batch_idx is not None, "batch_idx is required for paged kv cache"
        assert batch_idx.ndim in [1, 2], "batch_idx must be 1D (decode) or 2D (prefill 1xL)"
        self.flush()
        if batch_idx.ndim == 1:
            return self.assign(layer_id, batch_idx, input_pos, k, v)
        return self.assign_prefill_no_paging(layer_id, k, v, input_pos, batch_idx)

    def assign(self, layer_id: int, batch_idx: Tensor, input_pos: Tensor, k_val: Tensor, v_val: Tensor):
        """Decode append (:184-232): k_val, v_val [B, H, S, D] go to the slots of
        (batch_idx[b], input_pos[b, s]); unmapped (-1) pages are redirected to the
        reserved page 0.  Returns the layer's whole K and V pools, [1, H, N, D] views."""
        B, H, S, K_D = k_val.shape
        _, _, _, H_cache, MAX_S, D_cache = self.kv_shape
        assert H_cache == H, "number of heads must match"
        assert MAX_S >= S, "cache must have enough space"
        assert D_cache == K_D, "hidden dim must match"
        assert input_pos.shape == (B, S), "input_pos must have the same shape as val"
        assert batch_idx.shape == (B,), "batch_idx must have one dimension only"
        self.flush()
        if self.fuse_decode_append and S == 1 and k_val.dtype == self.dtype and v_val.dtype == self.dtype:
            # the attention call of this layer appends the rows itself (compiled_flex_attn_decode)
            self.last_decode_step = StepMeta(layer_id, input_pos, batch_idx, k_val, v_val)
            return self._pools[layer_id]
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
        self.flush()
        if self._kv_rep_unverified:
            self._check_v_copies(v_val)
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
        self.flush()
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

    def _check_v_copies(self, v_val: Tensor) -> None:
        """`kv_rep` > 1 that came from the class default, not from this cache's creator, is a claim about a
        model this cache may not belong to (a second engine in the process, a model without head repeat):
        the V rows of the first prefill step are compared inside each group, once, and a cache whose heads
        differ refuses to go on instead of decoding through the shared-V read (one wait for the stream)."""
        self._kv_rep_unverified = False
        H = v_val.shape[1]
        groups = v_val.reshape(v_val.shape[0], H // self.kv_rep, self.kv_rep, *v_val.shape[2:])
        if not bool((groups == groups[:, :, :1]).all()):
            raise RuntimeError(
                f"this cache took kv_rep={self.kv_rep} from install(kv_rep=...), but the V heads it is given are not "
                f"{self.kv_rep} identical copies per group; create it with PagedKVCache(..., kv_rep=1) or call "
                "install(kv_rep=1) before the engine that owns it is built")

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
        # a table narrower than the pool (max_blocks_per_seq) can be full while pages are free; with the
        # reference's dense table the pool always runs out first and its message is the one raised
        in_table = have // self.page_size + n_new <= self.table_cols
        if dry_run:
            return fits and in_table
        if not fits:
            raise RuntimeError(
                f"Cannot reserve {n_new} pages for a sequence of length {seq_len} "
                f"in batch {batch_idx_int}. Only {self.num_free_pages} pages available. "
                f"Current capacity is {have} tokens."
            )
        if not in_table:
            raise RuntimeError(
                f"Cannot reserve a sequence of length {seq_len} in batch {batch_idx_int}: "
                f"the page table holds {self.table_cols} blocks of {self.page_size} tokens per sequence."
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
        self.flush()
        self.check_prefill_masks(wait=False)
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
                                 BLOCK_SIZE: int = 128, *, open_spans=None,
                                 validate: bool | str = "deferred") -> HybridPrefillMask:
        """Mask of a packed prefill step: document-causal OR image-prefix (:343-362).

        `open_spans` and `validate` are not arguments of the reference.  `open_spans` lists the cache slots
        whose chunk begins inside an image span that an earlier chunk opened.  The row-limit kernel reports
        packed rows for which one limit per row is not the reference's mask (an end-of-image token with no
        span open; a span still open where the document changes or the row ends), and `validate` says when
        the host looks at that report:
          "deferred" (default)  the word travels to pinned host memory behind the kernel and is looked at by
                     the next `create_prefill_blockmask`, `erase` or `check_prefill_masks` -- no wait in this
                     call, as the reference's mask construction has none (its engine waits once per step,
                     `paged_inference.py:1083`).  A span open across a boundary then raises RuntimeError one
                     step late; a stray end-of-image token only warns, because the limits the kernel wrote for
                     it are the reference's own mask (which counts delimiters over the whole packed row,
                     `attention.py:75-96`) unless the caller is prefilling in chunks;
          True       this call waits for the kernel and raises for either report: for callers that prefill in
                     chunks (an undeclared chunk start inside a span) and for tests;
          False      nobody looks."""
        assert batch_idx.ndim == 2 and batch_idx.shape[0] == 1
        self.flush()
        self.check_prefill_masks(wait=True)  # the report of the step before: landed long ago
        return HybridPrefillMask(self, batch_idx, input_ids, soi_id, eoi_id, BLOCK_SIZE,
                                 open_spans=open_spans, validate=validate)

    _MASK_REPORTS = (
        "an end-of-image token closes a span that was not opened in this packed row; a chunk that starts inside "
        "an image span must be declared with open_spans=[slot]",
        "an image span is still open where batch_idx changes or the packed row ends; its rows would need keys of "
        "another sequence or keys that are not cached yet",
    )

    def _report_mask_status(self, bits: int, late: bool) -> None:
        when = "the previous create_prefill_blockmask" if late else "create_prefill_blockmask"
        if bits & 2:
            raise RuntimeError(f"{when}: {self._MASK_REPORTS[1]}")
        if bits & 1:
            if not late:
                raise RuntimeError(f"{when}: {self._MASK_REPORTS[0]}")
            warnings.warn(f"{when}: {self._MASK_REPORTS[0]} (the rows were masked as the reference masks them: "
                          "delimiters counted over the whole packed row)", RuntimeWarning, stacklevel=3)

    def _defer_mask_status(self, status: Tensor) -> None:
        """Send the status word of a row-limit launch to pinned host memory behind the kernel."""
        if self._mask_status_host is None:
            self._mask_status_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
            self._mask_status_event = torch.cuda.Event()
        self._mask_status_host.copy_(status, non_blocking=True)
        self._mask_status_event.record(torch.cuda.current_stream(status.device))
        self._mask_status_pending = True

    _mask_status_pending = False

    def check_prefill_masks(self, wait: bool = True) -> None:
        """Look at the report of the last deferred `create_prefill_blockmask` (see there).  `wait=False` looks
        only if the word has already arrived.  An engine calls this where it waits for the device anyway."""
        if not self._mask_status_pending:
            return
        if not wait and not self._mask_status_event.query():
            return
        self._mask_status_event.synchronize()
        self._mask_status_pending = False
        bits = int(self._mask_status_host[0])
        if bits:
            self._report_mask_status(bits, late=True)

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
            # sized for the largest batch and the longest context the page table can hold, at the finest split
            # either can get, so that later shapes fit.  Should one not (more query heads), the old buffer is
            # kept alive: graphs captured with it go on writing to it.
            worst_b = max(B, self.max_batch_size)
            worst_ctx = max(max_context, self.table_cols * self.page_size)
            need = 0
            for ctx in {max_context, worst_ctx}:
                finest = min(self.decode_split_tokens(1, Hc, ctx), self.decode_split_tokens(worst_b, Hc, ctx))
                need = max(need, ops.decode_workspace_bytes(worst_b, Hq, D, ctx, finest))
            if need and (self._workspace is None or self._workspace.numel() < need):
                if self._workspace is not None:
                    self._retired_workspaces.append(self._workspace)
                self._workspace = torch.empty(need, dtype=torch.uint8, device=self._kv.device)
            hit = (need, self.decode_split_tokens(B, Hc, max_context))
            self._decode_launch[key] = hit
        return (self._workspace if hit[0] else None), hit[1]

    def decode_plan(self) -> Tensor:
        """Buffer of the decode step's plan (`fp_paged_decode_plan`): allocated once, so that graphs captured
        with it stay valid.  `compiled_flex_attn_decode` writes it at the first layer of a step and the other
        layers of the step read it."""
        if self._decode_plan is None:
            self._decode_plan = torch.zeros(ops.decode_plan_bytes(), dtype=torch.uint8, device=self._kv.device)
        return self._decode_plan

    def score_bound(self, head_dim: int, scale: float | None) -> float:
        """Bound of |scale * q.k| the prefill kernel may rely on: 0 (unknown) unless q and k are normalised;
        then scale * head_dim with a tenth of slack for the roundings after the norm and the rotation."""
        if not self.qk_normalised:
            return 0.0
        return 1.1 * head_dim * (head_dim ** -0.5 if scale is None else abs(scale))

    def prefill_tile_rows(self, Lq: int, Hq: int, D: int, Hc: int, dtype: torch.dtype, workspace_bytes: int) -> int:
        """Rows per query tile of the prefill launch of this shape (`ops.prefill_tile_rows`), asked once per shape."""
        key = (Lq, Hq, Hc, D, dtype, workspace_bytes)
        hit = self._prefill_tile_rows.get(key)
        if hit is None:
            hit = self._prefill_tile_rows[key] = ops.prefill_tile_rows(Lq, Hq, Hc, D, dtype, workspace_bytes)
        return hit

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
            self._prefill_workspace = torch.empty(need, dtype=torch.uint8, device=self._kv.device)
        return self._prefill_workspace
