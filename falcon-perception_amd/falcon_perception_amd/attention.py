"""Attention entry points with the reference's names and call signature.

The reference binds `compiled_flex_attn_decode` / `compiled_flex_attn_prefill`
(`falcon_perception/attention.py:17-18`) in `model.py:20-24` and calls them as
`fn(q, k, v, block_mask=..., return_aux=AuxRequest(lse=True), kernel_options=...)`
(`model.py:156-162`).  Here the same names dispatch on the mask object:

* a `PagedDecodeMask` (what `PagedKVCache.convert_logical_block_mask` returns) runs
  the split-K paged decode kernel,
* a `HybridPrefillMask` (what `PagedKVCache.create_prefill_blockmask` returns) runs
  the MFMA chunked-prefill kernel over the paged cache,
* any other mask is not part of the paged path (the reference's AnyUp upsampler
  uses a windowed torch BlockMask, `anyup.py:358`) and is handed to torch's own
  flex_attention untouched.

The mask-mod factories and `create_attention_mask` keep the reference's names
(`attention.py:22-131`) because `paged_attention.py:16-20`, `model.py:23` and
`batch_inference.py:8` import them.
"""

from __future__ import annotations

import torch
from torch import Tensor
from torch.nn.attention.flex_attention import AuxOutput, BlockMask, and_masks, or_masks

from . import ops

__all__ = [
    "compiled_flex_attn_decode",
    "compiled_flex_attn_prefill",
    "create_attention_mask",
    "create_batch_attention_mask",
    "get_causal_mask_mod",
    "get_document_mask_mod",
    "get_image_prefix_mask_mod",
    "get_non_left_pad_mask_mod",
    "offset_mask_mod",
    "PagedDecodeMask",
    "HybridPrefillMask",
]


# --------------------------------------------------------------------------
# mask objects of the paged path
# --------------------------------------------------------------------------

class PagedDecodeMask:
    """Decode-step mask in physical page space.

    Returned by `PagedKVCache.convert_logical_block_mask`.  The decode kernel needs
    only the cache (page table), the batch rows and the positions of the step, so
    the physical block lists the reference materialises every step
    (`paged_attention.py:279-301`) are computed on first access only.
    """

    def __init__(self, cache, logical: BlockMask, batch_idx: Tensor):
        self.cache = cache
        self.logical = logical
        self.batch_idx = batch_idx
        self.BLOCK_SIZE = logical.BLOCK_SIZE
        self.seq_lengths = (logical.seq_lengths[0], cache.n_pages * cache.page_size)
        self._physical: dict[str, Tensor | None] = {}
        self._plan_shape = None  # launch shape the cache's decode plan was made for while this mask owned it

    @property
    def max_context(self) -> int:
        """Upper bound of the logical context length (KV length of the logical mask)."""
        return min(int(self.logical.seq_lengths[1]), self.cache.table_cols * self.cache.page_size)

    def _converted(self, name: str) -> Tensor | None:
        if name not in self._physical:
            src = getattr(self.logical, name)
            self._physical[name] = (
                None if src is None else ops.convert_block_ids(src, self.cache.page_table, self.batch_idx)
            )
        return self._physical[name]

    @property
    def kv_num_blocks(self) -> Tensor:
        return self.logical.kv_num_blocks.clone()

    @property
    def kv_indices(self) -> Tensor:
        return self._converted("kv_indices")

    @property
    def full_kv_num_blocks(self) -> Tensor | None:
        src = self.logical.full_kv_num_blocks
        return None if src is None else src.clone()

    @property
    def full_kv_indices(self) -> Tensor | None:
        return self._converted("full_kv_indices")

    @property
    def mask_mod(self):
        return self.cache.get_mask_mod(self.logical.mask_mod, self.batch_idx)

    def as_block_mask(self) -> BlockMask:
        """The torch BlockMask the reference would have built (`paged_attention.py:293-301`)."""
        return BlockMask.from_kv_blocks(
            self.kv_num_blocks, self.kv_indices, self.full_kv_num_blocks, self.full_kv_indices,
            self.BLOCK_SIZE, self.mask_mod, seq_lengths=self.seq_lengths,
        )


class HybridPrefillMask:
    """Prefill mask: document-causal OR bidirectional inside an image span.

    Returned by `PagedKVCache.create_prefill_blockmask`.  Holds, per packed row, the
    packed index one past the last key the row may see (`row_hi`); together with the
    row's own position this is the whole mask (`attention.py:75-96`,
    `paged_attention.py:353-359`).
    """

    def __init__(self, cache, batch_idx: Tensor, input_ids: Tensor, soi_id: int, eoi_id: int, block_size: int,
                 open_spans=None, validate: bool | str = "deferred", row_hi: Tensor | None = None):
        self.cache = cache
        self.batch_idx = batch_idx
        self.input_ids = input_ids
        self.soi_id = soi_id
        self.eoi_id = eoi_id
        self.BLOCK_SIZE = (block_size, block_size)
        L = batch_idx.shape[1]
        self.seq_lengths = (L, L)
        if row_hi is None:  # [L] int32, packed coordinates
            row_hi = self._limits_from_ids(open_spans, validate)
        self.row_hi = row_hi
        self._arange = torch.arange(L, dtype=torch.int64, device=batch_idx.device)
        self._step_key = None  # (address, shape) of the positions whose row limits are kept below
        self._step_layer = -1  # layer that asked last: a layer id that does not grow starts a new step
        self._row_limit = None
        self._tile_orders: dict[int, tuple[Tensor, int]] = {}  # rows per tile -> tile order of the step's limits

    def _limits_from_ids(self, open_spans, validate) -> Tensor:
        """Run the row-limit kernel and hand its report to the cache.

        The reference's `or_masks(image_prefix, document_causal)` (`paged_attention.py:350-361`) counts
        soi / eoi tokens over the whole packed row.  A span that is still open where the document changes
        would let its rows see the next document, and a chunk that starts inside a span has no soi to
        count: neither occurs in the reference's engine (whole sequences, `paged_inference.py:637-672`).
        `open_spans` (cache slots) declares the second case, which is then served: those rows are
        bidirectional up to the eoi.  When and how the kernel's report is looked at is `validate`
        (`PagedKVCache.create_prefill_blockmask`); only `validate=True` waits for the stream here."""
        if validate not in (True, False, "deferred"):
            raise ValueError('validate must be True, False or "deferred"')
        dev = self.batch_idx.device
        open_at_start = None
        if open_spans is not None:
            flags = torch.zeros(self.cache.max_batch_size, dtype=torch.uint8)
            for slot in open_spans:
                flags[int(slot)] = 1
            open_at_start = flags.to(dev)
        status = torch.zeros(1, dtype=torch.int32, device=dev) if validate else None
        row_hi = ops.hybrid_row_limits(self.input_ids, self.soi_id, self.eoi_id, self.batch_idx,
                                       open_at_start, status)
        if validate is True:
            bits = int(status.item())
            if bits:
                self.cache._report_mask_status(bits, late=False)
        elif validate == "deferred":
            self.cache._defer_mask_status(status)
        return row_hi

    def row_limit(self, input_pos: Tensor, layer_id: int = 0) -> Tensor:
        """Logical key limit of each row: its position plus the reach of `row_hi` beyond the row.

        Computed by the first layer of a step and kept for the layers after it (`layer_id` growing over
        the same positions tensor).  The key holds nothing that an inference tensor lacks: the reference's
        engine builds `input_pos` under `torch.inference_mode()` (`paged_inference.py:646-675, 1331`),
        where tensors carry no version counter."""
        key = (input_pos.data_ptr(), tuple(input_pos.shape), input_pos.dtype)
        if key != self._step_key or layer_id <= self._step_layer:
            reach = self.row_hi.to(torch.int64) - self._arange
            self._row_limit = (input_pos.reshape(-1) + reach).to(torch.int32)
            self._step_key = key
            self._tile_orders = {}
        self._step_layer = layer_id
        return self._row_limit

    def tile_order(self, batch_idx: Tensor, tile_rows: int) -> tuple[Tensor, int]:
        """Query tiles of the step by decreasing key range (`ops.prefill_tile_order`), made by the first layer
        that asks after `row_limit` and kept for the layers after it."""
        hit = self._tile_orders.get(tile_rows)
        if hit is None:
            hit = self._tile_orders[tile_rows] = ops.prefill_tile_order(batch_idx, self._row_limit, tile_rows)
        return hit


# --------------------------------------------------------------------------
# the two attention callables
# --------------------------------------------------------------------------

_torch_flex = {}


def _foreign(kind: str, q, k, v, kwargs):
    """Masks this package does not own go to torch's flex_attention unchanged."""
    if kind not in _torch_flex:
        from torch.nn.attention.flex_attention import flex_attention

        opts = {"fullgraph": True} if kind == "decode" else {"dynamic": True}
        _torch_flex[kind] = torch.compile(flex_attention, **opts)
    return _torch_flex[kind](q, k, v, **kwargs)


def _result(out: Tensor, lse: Tensor, return_aux, return_lse: bool):
    if return_aux is not None:
        want_lse = getattr(return_aux, "lse", False)
        return out, AuxOutput(lse=lse if want_lse else None)
    if return_lse:
        return out, lse
    return out


def compiled_flex_attn_decode(q: Tensor, k: Tensor, v: Tensor, score_mod=None, block_mask=None,
                              scale: float | None = None, enable_gqa: bool = False,
                              return_lse: bool = False, kernel_options=None, *, return_aux=None,
                              sinks: Tensor | None = None):
    """Decode attention, one query token per sequence (`attention.py:17`, `model.py:156-162`).

    q [B, Hq, 1, D]; k, v are the pool views `PagedKVCache.insert_kv` returned,
    [1, Hc, n_slots, D].  `kernel_options` are Triton tuning knobs of the reference
    and are ignored.  `sinks` [Hq] float32 (not an argument of the reference's callable) applies
    the sink gate of `Attention._post_attention` (`model.py:122-126`) to the returned output.

    The kernel attends positions 0 .. input_pos[b] of every sequence, i.e. the causal mask the engine
    installs for a decode step (`q + input_pos[b] >= kv`, `paged_inference.py:797-801`); the `mask_mod` of
    the logical mask is not evaluated, so a mask that hides earlier positions is outside this path.
    """
    if not isinstance(block_mask, PagedDecodeMask):
        if sinks is not None:
            raise RuntimeError("the fused sink gate needs a mask made by PagedKVCache")
        return _foreign("decode", q, k, v, dict(score_mod=score_mod, block_mask=block_mask, scale=scale,
                                                enable_gqa=enable_gqa, return_lse=return_lse,
                                                kernel_options=kernel_options, return_aux=return_aux))
    if score_mod is not None:
        raise RuntimeError("score_mod is not supported on the paged decode path")
    cache = block_mask.cache
    step = cache.last_decode_step
    if step is None:
        raise RuntimeError("paged decode attention called before PagedKVCache.insert_kv for this step")
    if q.shape[2] != 1:
        raise RuntimeError("a PagedDecodeMask serves one query token per sequence")
    if step.batch_idx.shape != block_mask.batch_idx.shape:
        raise RuntimeError(
            f"the mask was converted for {tuple(block_mask.batch_idx.shape)} sequences but the last insert_kv of this "
            f"cache appended {tuple(step.batch_idx.shape)}: attention must follow the insert_kv of its own step")
    kv_rep = getattr(cache, "kv_rep", 1)
    wg_heads = k.shape[1] // kv_rep  # workgroups per sequence and split
    workspace, split_tokens = cache.decode_launch(q.shape[0], q.shape[1], q.shape[3], block_mask.max_context, wg_heads)
    # the pool views insert_kv returned, as planes [H, N, D]: the cache keeps both forms of every layer
    pools = cache._pools[step.layer_id]
    own = k is pools[0] and v is pools[1]
    pool_k, pool_v = cache._planes[step.layer_id] if own else (k[0], v[0])
    k_new = v_new = None
    if step.k_new is not None:
        # the append of this step was left to this launch (`PagedKVCache.fuse_decode_append`): the kernel
        # appends the rows and attends over them.  Any other k, v than the pool views of the step's layer
        # means the caller is not the model's insert -> attend pair, and the plain append runs first.
        if own and step.k_new.shape[0] == q.shape[0]:
            k_new, v_new = step.k_new, step.v_new
            cache.last_decode_step = step._replace(k_new=None, v_new=None)
        else:
            cache.flush()
    # The plan of the step: the reference converts its mask once per step and every layer consumes it
    # (paged_inference.py:847-848, model.py:689-699); here the first attention call that meets this mask object
    # has the decode kernel's per-step work done once, and the layers after it start from the result.
    plan = cache.decode_plan()
    args = (q, pool_k, pool_v, cache.page_table, block_mask.batch_idx, step.input_pos, cache.page_size,
            block_mask.max_context)
    shape = (q.shape[0], q.shape[1], q.shape[3], k.shape[1], kv_rep, split_tokens, step.input_pos.data_ptr())
    if cache._decode_plan_owner is not block_mask or block_mask._plan_shape != shape:
        ops.paged_decode(*args, scale=scale, split_tokens=split_tokens, kv_rep=kv_rep, phase="plan", plan=plan)
        cache._decode_plan_owner = block_mask
        block_mask._plan_shape = shape
    out, lse = ops.paged_decode(*args, scale=scale, workspace=workspace, split_tokens=split_tokens, sinks=sinks,
                                kv_rep=kv_rep, k_new=k_new, v_new=v_new, plan=plan)
    return _result(out, lse, return_aux, return_lse)


def compiled_flex_attn_prefill(q: Tensor, k: Tensor, v: Tensor, score_mod=None, block_mask=None,
                               scale: float | None = None, enable_gqa: bool = False,
                               return_lse: bool = False, kernel_options=None, *, return_aux=None,
                               sinks: Tensor | None = None):
    """Prefill attention over the paged cache under the hybrid mask (`attention.py:18`).

    q [1, Hq, L, D] packed rows.  Keys and values are read from the pages that
    `PagedKVCache.insert_kv` has just filled for this layer (the k, v arguments are
    the fresh rows it returned and are not read again), so a chunk whose prefix
    already lives in pages attends over prefix and chunk alike.
    """
    if not isinstance(block_mask, HybridPrefillMask):
        if sinks is not None:
            raise RuntimeError("the fused sink gate needs a mask made by PagedKVCache")
        return _foreign("prefill", q, k, v, dict(score_mod=score_mod, block_mask=block_mask, scale=scale,
                                                 enable_gqa=enable_gqa, return_lse=return_lse,
                                                 kernel_options=kernel_options, return_aux=return_aux))
    if score_mod is not None:
        raise RuntimeError("score_mod is not supported on the paged prefill path")
    cache = block_mask.cache
    cache.flush()
    step = cache.last_prefill_step
    if step is None:
        raise RuntimeError("paged prefill attention called before PagedKVCache.insert_kv for this step")
    pool_k, pool_v = cache._planes[step.layer_id]
    Lq, Hq, D = q.shape[2], q.shape[1], q.shape[3]
    limits = block_mask.row_limit(step.input_pos, step.layer_id)
    workspace = cache.prefill_workspace(Lq, Hq, D, pool_k.shape[0], q.dtype)
    # At head_dim 64 several small workgroups share a CU and the order in which they start decides when the launch
    # ends: the step's query tiles are ranked once (first layer) and every layer starts the longest first.  At
    # head_dim 128 the order measured no difference, so no kernel is spent on it.
    order = None
    if D == 64:
        rows = cache.prefill_tile_rows(Lq, Hq, D, pool_k.shape[0], q.dtype, workspace.numel() if workspace is not False else 0)
        if rows and -(-Lq // rows) <= 4096:
            order = block_mask.tile_order(step.batch_idx, rows)
    out, lse = ops.paged_prefill(
        q, pool_k, pool_v, cache.page_table, step.batch_idx, limits, cache.page_size, scale=scale, sinks=sinks,
        workspace=workspace, score_bound=cache.score_bound(D, scale), tile_order=order,
    )
    return _result(out, lse, return_aux, return_lse)


# --------------------------------------------------------------------------
# mask-mod factories (names of attention.py:22-131)
# --------------------------------------------------------------------------

def offset_mask_mod(mask_mod, offset: int):
    """mask_mod evaluated with the query index shifted by `offset` (`attention.py:22-28`)."""
    return lambda b, h, q, kv: mask_mod(b, h, q + offset, kv)


def get_causal_mask_mod():
    """kv may not lie after q (`attention.py:31-37`)."""
    return lambda b, h, q_idx, kv_idx: q_idx >= kv_idx


def get_document_mask_mod(batch: Tensor, eos_id: int):
    """Tokens attend only inside their own eos-delimited document (`attention.py:40-60`)."""
    ends = batch == eos_id
    ends[:, -1] = True
    closed = torch.cumsum(ends.to(torch.int32), dim=1)
    doc_id = torch.zeros_like(closed, dtype=torch.int32)
    doc_id[:, 1:] = closed[:, :-1]
    return lambda b, h, q_idx, kv_idx: doc_id[b, q_idx] == doc_id[b, kv_idx]


def get_non_left_pad_mask_mod(batch: Tensor, pad_id: int):
    """Keys that are left padding are never attended (`attention.py:63-72`)."""
    seen_real = torch.cumsum(batch != pad_id, dim=1)
    return lambda b, h, q_idx, kv_idx: seen_real[b, kv_idx] > 0


def get_image_prefix_mask_mod(batch: Tensor, soi_id: int, eoi_id: int):
    """Bidirectional attention between tokens of one image span (`attention.py:75-96`)."""
    opened = torch.cumsum(batch == soi_id, dim=1)
    closed = torch.cumsum(batch == eoi_id, dim=1)
    inside = (opened - closed) > 0
    span = opened * inside
    return lambda b, h, q_idx, kv_idx: (inside[b, q_idx] & inside[b, kv_idx]) & (span[b, q_idx] == span[b, kv_idx])


@torch.inference_mode()
def create_attention_mask(*args, **kwargs) -> BlockMask:
    """torch `create_block_mask` under inference mode (`attention.py:99-102`).

    Only masks outside the paged path are built this way (the dense batch engine);
    the paged path builds its masks in closed form in `paged_attention.py`.
    """
    from torch.nn.attention.flex_attention import create_block_mask

    return create_block_mask(*args, **kwargs)


def create_batch_attention_mask(input_batch: Tensor, *, pad_token_id: int, eos_token_id: int,
                                soi_token_id: int, eoi_token_id: int, max_len: int | None = None) -> BlockMask:
    """Mask of the dense batch engine (`attention.py:105-131`): image-prefix OR (causal AND document AND non-left-pad)."""
    B, S = input_batch.size()
    text = and_masks(get_causal_mask_mod(), get_document_mask_mod(input_batch, eos_token_id),
                     get_non_left_pad_mask_mod(input_batch, pad_token_id))
    image = get_image_prefix_mask_mod(input_batch, soi_token_id, eoi_token_id)
    n = max_len or S
    return create_attention_mask(or_masks(image, text), B, None, n, n)
