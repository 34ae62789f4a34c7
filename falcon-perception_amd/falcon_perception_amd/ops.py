"""Tensor-level wrappers of the C ABI: torch supplies device memory and the stream,
the HIP kernels of libfp_paged_kv.so do the work.  No wrapper allocates unless the
caller leaves an output or workspace argument out, and none synchronises.
"""

from __future__ import annotations

import math

import torch
from torch import Tensor

from . import _native as N


def _rows(t: Tensor) -> Tensor:
    """Make the head_dim axis dense (the kernels move whole rows)."""
    return t if t.stride(-1) == 1 else t.contiguous()


def kv_append(pool_k: Tensor, pool_v: Tensor, k: Tensor, v: Tensor, page_table: Tensor,
              batch_idx: Tensor, input_pos: Tensor, page_size: int, clamp_negative: bool,
              packed: bool = False) -> None:
    """Scatter k, v [T, H, S, D] into pool_k, pool_v [H, N, D] at the slots the page table gives.

    batch_idx [T] int64, input_pos [T, S] int32/int64.  Byte-exact copy
    (reference paged_attention.py:212-230 with clamp, :387-391 without).
    `packed`: k, v are the prefill layout [1, H, L, D] with batch_idx, input_pos [1, L]; they are read as
    L row groups of one token each through their strides.
    """
    N.require_cuda(pool_k, pool_v, k, v, page_table, batch_idx, input_pos)
    if v.shape != k.shape:
        raise RuntimeError(f"k {tuple(k.shape)} and v {tuple(v.shape)} must have the same shape")
    if pool_k.dtype != k.dtype or pool_v.dtype != v.dtype:
        raise RuntimeError(f"dtype mismatch: pool {pool_k.dtype}, k {k.dtype}, v {v.dtype}")
    if not (pool_k.is_contiguous() and pool_v.is_contiguous()):
        raise RuntimeError("pool planes must be contiguous [H, N, D]")
    k, v = _rows(k), _rows(v)
    if packed:
        one, H, T, D = k.shape
        S = 1
        if one != 1 or batch_idx.numel() != T or input_pos.numel() != T:
            raise RuntimeError("packed rows are [1, H, L, D] with L entries of batch_idx and input_pos")
        ks, vs = (k.stride(2), k.stride(1), 0), (v.stride(2), v.stride(1), 0)
    else:
        T, H, S, D = k.shape
        ks, vs = (k.stride(0), k.stride(1), k.stride(2)), (v.stride(0), v.stride(1), v.stride(2))
    if not input_pos.is_contiguous():
        input_pos = input_pos.contiguous()
    if not batch_idx.is_contiguous():
        batch_idx = batch_idx.contiguous()
    if batch_idx.dtype != torch.int64:
        batch_idx = batch_idx.to(torch.int64)
    if page_table.dtype != torch.int64 or page_table.stride(1) != 1:
        raise RuntimeError("page_table must be int64 with a dense last axis")
    rc = N.lib().fp_kv_append(
        pool_k.data_ptr(), pool_v.data_ptr(), k.data_ptr(), v.data_ptr(), *ks, *vs,
        page_table.data_ptr(), page_table.stride(0), batch_idx.data_ptr(),
        input_pos.data_ptr(), N.index_code(input_pos),
        T, H, S, D, page_size, page_table.shape[1], page_table.shape[0],
        pool_k.shape[1], N.dtype_code(k.dtype), int(clamp_negative), N.stream_ptr(k.device))
    N.check(rc, "fp_kv_append")


def qkv_norm_rope_append(xq: Tensor, xk: Tensor, xv: Tensor, freqs_cis: Tensor, freqs_cis_2d: Tensor | None,
                         pool_k: Tensor, pool_v: Tensor, page_table: Tensor, batch_idx: Tensor, input_pos: Tensor,
                         page_size: int, *, eps: float | None = None, clamp_negative: bool = True,
                         q_out: Tensor | None = None) -> Tensor:
    """RMS norm of q and k, head repeat, 3D rotary embedding and the cache insert in one launch
    (reference `model.py:110-119` + `paged_attention.py:184-232, 364-393`).

    xq [B, S, Hq, D], xk / xv [B, S, Hkv, D] (views of the qkv projection are fine); freqs_cis
    [B, S, D/4] complex64, freqs_cis_2d None or [B, S, Hq, D/4] complex64; batch_idx and input_pos
    one entry per token ([B*S] after flattening).  Returns the rotated q as [B, Hq, S, D]."""
    N.require_cuda(xq, xk, xv, freqs_cis, freqs_cis_2d, pool_k, pool_v, page_table, batch_idx, input_pos, q_out)
    B, S, Hq, D = xq.shape
    Hkv = xk.shape[2]
    if xk.shape != (B, S, Hkv, D) or xv.shape != xk.shape or xk.dtype != xq.dtype or xv.dtype != xq.dtype:
        raise RuntimeError("xq / xk / xv shape or dtype mismatch")
    if B > 1 and S > 1:
        raise RuntimeError("one of batch and sequence must be 1 (decode [B, 1, ..] or packed prefill [1, L, ..])")
    H_pool, n_slots, Dp = pool_k.shape
    if Dp != D or pool_v.shape != pool_k.shape or pool_k.dtype != xq.dtype or pool_v.dtype != xq.dtype:
        raise RuntimeError("pool shape or dtype mismatch")
    T = B * S

    def rows(x):  # [B, S, H, D] -> (tensor, token stride, head stride) with one stride for all tokens
        if x.stride(3) != 1:
            x = x.contiguous()
        return x, (x.stride(1) if S > 1 else x.stride(0)), x.stride(2)

    xq, qs_t, qs_h = rows(xq)
    xk, ks_t, ks_h = rows(xk)
    xv, vs_t, vs_h = rows(xv)
    if freqs_cis.dtype != torch.complex64 or freqs_cis.shape != (B, S, D // 4):
        raise RuntimeError("freqs_cis must be complex64 of shape [B, S, D/4]")
    f1 = torch.view_as_real(freqs_cis.contiguous())
    f2 = None
    if freqs_cis_2d is not None:
        if freqs_cis_2d.dtype != torch.complex64 or freqs_cis_2d.shape != (B, S, Hq, D // 4):
            raise RuntimeError("freqs_cis_2d must be complex64 of shape [B, S, Hq, D/4]")
        f2 = torch.view_as_real(freqs_cis_2d.contiguous())
    batch_idx = batch_idx.reshape(-1).contiguous()
    input_pos = input_pos.reshape(-1).contiguous()
    if batch_idx.dtype != torch.int64 or batch_idx.shape[0] != T or input_pos.shape[0] != T:
        raise RuntimeError("batch_idx (int64) and input_pos need one entry per token")
    if q_out is None:
        q_out = torch.empty((B, Hq, S, D), dtype=xq.dtype, device=xq.device)
    if q_out.shape != (B, Hq, S, D) or q_out.stride(3) != 1:
        raise RuntimeError("q_out must be [B, Hq, S, D] with dense rows")
    if eps is None:
        eps = torch.finfo(torch.float32).eps  # F.rms_norm(eps=None): epsilon of the fp32 computation type
    rc = N.lib().fp_qkv_norm_rope_append(
        xq.data_ptr(), xk.data_ptr(), xv.data_ptr(), qs_t, qs_h, ks_t, ks_h, vs_t, vs_h,
        f1.data_ptr(), f2.data_ptr() if f2 is not None else None,
        q_out.data_ptr(), q_out.stride(2) if S > 1 else q_out.stride(0), q_out.stride(1),
        pool_k.data_ptr(), pool_v.data_ptr(), page_table.data_ptr(), page_table.stride(0),
        batch_idx.data_ptr(), input_pos.data_ptr(), N.index_code(input_pos),
        T, Hq, Hkv, H_pool, D, page_size, page_table.shape[1], page_table.shape[0], n_slots,
        float(eps), N.dtype_code(xq.dtype), 1 if clamp_negative else 0, N.stream_ptr(xq.device))
    N.check(rc, "fp_qkv_norm_rope_append")
    return q_out


def kv_gather(pool: Tensor, page_table: Tensor, batch_idx: Tensor, seq_lens: Tensor,
              page_size: int, max_len: int, out: Tensor | None = None) -> Tensor:
    """Dense logical view [B, H, max_len, D] of the cached rows of each sequence; zero tail."""
    N.require_cuda(pool, page_table, batch_idx, seq_lens, out)
    H, n_slots, D = pool.shape
    B = batch_idx.shape[0]
    if out is None:
        out = torch.empty((B, H, max_len, D), dtype=pool.dtype, device=pool.device)
    elif out.shape != (B, H, max_len, D) or out.dtype != pool.dtype or out.stride(3) != 1:
        raise RuntimeError("out must be [B, H, max_len, D] of the pool dtype with dense rows")
    batch_idx = batch_idx.contiguous()
    seq_lens = seq_lens.contiguous()
    rc = N.lib().fp_kv_gather(
        pool.data_ptr(), out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
        page_table.data_ptr(), page_table.stride(0), batch_idx.data_ptr(),
        seq_lens.data_ptr(), N.index_code(seq_lens),
        B, H, max_len, D, page_size, page_table.shape[1], page_table.shape[0],
        n_slots, N.dtype_code(pool.dtype), N.stream_ptr(pool.device))
    N.check(rc, "fp_kv_gather")
    return out


def convert_block_ids(kv_indices: Tensor, page_table: Tensor, batch_idx: Tensor) -> Tensor:
    """kv_indices [B, H, R, C] int32 logical blocks -> [B, H, R, n_pages] int32 physical pages."""
    N.require_cuda(kv_indices, page_table, batch_idx)
    B, H, R, C = kv_indices.shape
    n_pages = page_table.shape[1]
    if kv_indices.dtype != torch.int32:
        kv_indices = kv_indices.to(torch.int32)
    kv_indices = kv_indices.contiguous()
    batch_idx = batch_idx.contiguous()
    out = torch.empty((B, H, R, n_pages), dtype=torch.int32, device=kv_indices.device)
    rc = N.lib().fp_convert_block_ids(
        kv_indices.data_ptr(), out.data_ptr(), page_table.data_ptr(), page_table.stride(0),
        batch_idx.data_ptr(), B, H * R, C, n_pages, page_table.shape[0],
        N.stream_ptr(kv_indices.device))
    N.check(rc, "fp_convert_block_ids")
    return out


def decode_split_tokens(B: int, Hc: int, max_context: int, page_size: int) -> int:
    return int(N.lib().fp_paged_decode_default_split(B, Hc, max_context, page_size))


def decode_workspace_bytes(B: int, Hq: int, D: int, max_context: int, split_tokens: int) -> int:
    n = int(N.lib().fp_paged_decode_workspace_bytes(B, Hq, D, max_context, split_tokens))
    N.check(n, "fp_paged_decode_workspace_bytes")
    return n


def _sinks_ptr(sinks: Tensor | None, Hq: int, device) -> int | None:
    if sinks is None:
        return None
    N.require_cuda(sinks)
    if sinks.dtype != torch.float32 or sinks.shape != (Hq,) or not sinks.is_contiguous() or sinks.device != device:
        raise RuntimeError("sinks must be a contiguous float32 tensor of shape [Hq] on the device of q")
    return sinks.data_ptr()


def paged_decode(q: Tensor, pool_k: Tensor, pool_v: Tensor, page_table: Tensor, batch_idx: Tensor,
                 input_pos: Tensor, page_size: int, max_context: int, *, scale: float | None = None,
                 split_tokens: int = 0, workspace: Tensor | None = None,
                 out: Tensor | None = None, lse: Tensor | None = None, phase: str = "both",
                 k_new: Tensor | None = None, v_new: Tensor | None = None,
                 sinks: Tensor | None = None, kv_rep: int = 1, plan: Tensor | None = None) -> tuple[Tensor, Tensor]:
    """Single-query paged attention.  q [B, Hq, 1, D]; pools [Hc, N, D]; returns out [B, Hq, 1, D], lse [B, Hq, 1].

    `kv_rep` > 1 declares a cache with one head per query head whose V heads are `kv_rep` identical
    copies (the reference's `repeat_kv` layout, `model.py:112-114`): V is then read once per group.

    With `sinks` [Hq] float32 the output is gated as the reference's `_post_attention` does
    (model.py:122-128): out * sigmoid(lse - sinks[h]); lse is returned ungated.

    With `k_new`, `v_new` [B, Hc, 1, D] the call is the whole decode step: the rows are appended at
    `input_pos` (as `kv_append` with clamp would) and attended over in the same launch.

    `phase` = "both" (default), "partial" (split-K pass only, results stay in `workspace`),
    "merge" (cross-split merge of a previous partial pass with the same arguments) or "plan" (write the
    step's plan into `plan` and launch nothing else).

    `plan`: a uint8 tensor of `decode_plan_bytes()` bytes.  Written by a `phase="plan"` call with the
    arguments of the step (once per step: the positions and page tables of all layers are the same), it lets
    the workgroups of a large launch start from one load instead of positions -> cut -> page table; results
    are bit-identical with and without."""
    N.require_cuda(q, pool_k, pool_v, page_table, batch_idx, input_pos, workspace, out, lse)
    B, Hq, Sq, D = q.shape
    if Sq != 1:
        raise RuntimeError(f"paged_decode takes one query token per sequence, got {Sq}")
    Hc, n_slots, Dp = pool_k.shape
    if Dp != D or pool_v.shape != pool_k.shape or pool_k.dtype != q.dtype or pool_v.dtype != q.dtype:
        raise RuntimeError("q / pool shape or dtype mismatch")
    q = _rows(q)
    input_pos = input_pos.reshape(-1).contiguous()
    batch_idx = batch_idx.contiguous()
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if input_pos.numel() != B or batch_idx.numel() != B:
        raise RuntimeError(f"input_pos ({input_pos.numel()}) and batch_idx ({batch_idx.numel()}) need one entry "
                           f"per sequence of q ({B})")
    if split_tokens == 0:
        split_tokens = decode_split_tokens(B, Hc // kv_rep if kv_rep > 1 else Hc, max_context, page_size)
    planning = phase == "plan"  # writes the plan only: no workspace, no results
    if workspace is None and not planning:  # a workspace the caller brings is checked by the library against the launch
        need = decode_workspace_bytes(B, Hq, D, max_context, split_tokens)
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
    if out is None and not planning:
        out = torch.empty((B, Hq, 1, D), dtype=q.dtype, device=q.device)
    if lse is None and not planning:
        lse = torch.empty((B, Hq, 1), dtype=torch.float32, device=q.device)
    if not planning and (out.stride(3) != 1 or not lse.is_contiguous() or lse.dtype != torch.float32):
        raise RuntimeError("out rows must be dense and lse contiguous float32")
    sinks_ptr = _sinks_ptr(sinks, Hq, q.device)
    entry = {"both": "fp_paged_decode", "partial": "fp_paged_decode_partial", "merge": "fp_paged_decode_merge",
             "plan": "fp_paged_decode_plan"}[phase]
    plan_ptr, plan_bytes = None, 0
    if plan is not None:
        N.require_cuda(plan)
        if plan.dtype != torch.uint8 or not plan.is_contiguous():
            raise RuntimeError("plan must be a contiguous uint8 tensor")
        plan_ptr, plan_bytes = plan.data_ptr(), plan.numel()
    elif phase == "plan":
        raise RuntimeError('phase="plan" needs the plan tensor to write')
    fresh = ()
    if k_new is not None or v_new is not None:
        if phase != "both" or k_new is None or v_new is None:
            raise RuntimeError("the fused append needs both k_new and v_new and runs both passes")
        N.require_cuda(k_new, v_new)
        if k_new.shape != (B, Hc, 1, D) or v_new.shape != (B, Hc, 1, D) or k_new.dtype != q.dtype or v_new.dtype != q.dtype:
            raise RuntimeError("k_new / v_new must be [B, Hc, 1, D] of the q dtype")
        k_new, v_new = _rows(k_new), _rows(v_new)
        entry = "fp_paged_decode_append"
        fresh = (k_new.data_ptr(), v_new.data_ptr(), k_new.stride(0), k_new.stride(1), v_new.stride(0), v_new.stride(1))
    rc = getattr(N.lib(), entry)(
        *fresh,
        q.data_ptr(), q.stride(0), q.stride(1), pool_k.data_ptr(), pool_v.data_ptr(),
        page_table.data_ptr(), page_table.stride(0), batch_idx.data_ptr(),
        input_pos.data_ptr(), N.index_code(input_pos),
        out.data_ptr() if out is not None else None, out.stride(0) if out is not None else 0,
        out.stride(1) if out is not None else 0, lse.data_ptr() if lse is not None else None, sinks_ptr,
        workspace.data_ptr() if workspace is not None else None,
        workspace.numel() * workspace.element_size() if workspace is not None else 0,
        B, Hq, Hc, kv_rep, D, page_size, page_table.shape[1], page_table.shape[0],
        n_slots, max_context, split_tokens, scale, N.dtype_code(q.dtype), plan_ptr, plan_bytes, N.stream_ptr(q.device))
    N.check(rc, entry)
    return out, lse


def decode_plan_bytes() -> int:
    """Bytes a decode plan buffer needs on the current device."""
    return int(N.lib().fp_paged_decode_plan_bytes())


def paged_decode_noalloc(q: Tensor, pool_k: Tensor, pool_v: Tensor, page_table: Tensor, batch_idx: Tensor,
                         input_pos: Tensor, page_size: int, max_context: int, out: Tensor, lse: Tensor, *,
                         scale: float | None = None, split_tokens: int = 0, sinks: Tensor | None = None,
                         kv_rep: int = 1) -> tuple[Tensor, Tensor]:
    """`paged_decode` for callers that may not allocate: the caller brings `out` [B, Hq, 1, D] and `lse`
    [B, Hq, 1], the split-K partial results go to an array inside the library (`_native.NOALLOC_SCRATCH_BYTES`;
    a larger launch raises), and neither this wrapper nor the library allocates.  Calls that overlap on one
    GPU share that array and race."""
    N.require_cuda(q, pool_k, pool_v, page_table, batch_idx, input_pos, out, lse)
    B, Hq, Sq, D = q.shape
    Hc, n_slots, Dp = pool_k.shape
    if Sq != 1 or Dp != D or pool_v.shape != pool_k.shape or pool_k.dtype != q.dtype or pool_v.dtype != q.dtype:
        raise RuntimeError("q / pool shape or dtype mismatch")
    if q.stride(3) != 1 or not input_pos.is_contiguous() or not batch_idx.is_contiguous():
        raise RuntimeError("q rows, input_pos and batch_idx must be dense (nothing is copied here)")
    if input_pos.numel() != B or batch_idx.numel() != B:
        raise RuntimeError("input_pos and batch_idx need one entry per sequence of q")
    if out.shape != (B, Hq, 1, D) or out.dtype != q.dtype or out.stride(3) != 1:
        raise RuntimeError("out must be [B, Hq, 1, D] of the q dtype with dense rows")
    if lse.shape != (B, Hq, 1) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise RuntimeError("lse must be contiguous float32 [B, Hq, 1]")
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    rc = N.lib().fp_paged_decode_noalloc(
        q.data_ptr(), q.stride(0), q.stride(1), pool_k.data_ptr(), pool_v.data_ptr(),
        page_table.data_ptr(), page_table.stride(0), batch_idx.data_ptr(),
        input_pos.data_ptr(), N.index_code(input_pos),
        out.data_ptr(), out.stride(0), out.stride(1), lse.data_ptr(), _sinks_ptr(sinks, Hq, q.device),
        B, Hq, Hc, kv_rep, D, page_size, page_table.shape[1], page_table.shape[0],
        n_slots, max_context, split_tokens, scale, N.dtype_code(q.dtype), N.stream_ptr(q.device))
    N.check(rc, "fp_paged_decode_noalloc")
    return out, lse


def hybrid_row_limits(input_ids: Tensor, soi_id: int, eoi_id: int, batch_idx: Tensor | None = None,
                      open_at_start: Tensor | None = None, status: Tensor | None = None) -> Tensor:
    """Packed index one past the last key each packed row may see: max(q + 1, end of q's image span).

    `batch_idx` [L] int64 names the document of every packed row, `open_at_start` [max_batch] uint8 the
    slots whose rows begin inside an image span opened by an earlier chunk.  `status` (one int32, written
    by the kernel) reports inputs for which one limit per row is not the reference's mask: bit 0 an eoi
    with no span open, bit 1 a span open across a document boundary or the end of the row."""
    N.require_cuda(input_ids, batch_idx, open_at_start, status)
    ids = input_ids.reshape(-1).contiguous()
    if ids.dtype != torch.int64:
        ids = ids.to(torch.int64)
    L = ids.shape[0]
    docs_ptr = open_ptr = status_ptr = None
    max_batch = 0
    if batch_idx is not None:
        batch_idx = batch_idx.reshape(-1).contiguous()
        if batch_idx.dtype != torch.int64 or batch_idx.shape[0] != L:
            raise RuntimeError("batch_idx must be int64 with one entry per packed row")
        docs_ptr = batch_idx.data_ptr()
    if open_at_start is not None:
        if batch_idx is None or open_at_start.dtype != torch.uint8 or not open_at_start.is_contiguous():
            raise RuntimeError("open_at_start must be a contiguous uint8 tensor and needs batch_idx")
        open_ptr, max_batch = open_at_start.data_ptr(), open_at_start.numel()
    if status is not None:
        if status.dtype != torch.int32 or status.numel() != 1:
            raise RuntimeError("status must hold one int32")
        status_ptr = status.data_ptr()
    out = torch.empty(L, dtype=torch.int32, device=ids.device)
    rc = N.lib().fp_hybrid_row_limits(ids.data_ptr(), docs_ptr, open_ptr, max_batch, L, soi_id, eoi_id,
                                      out.data_ptr(), status_ptr, N.stream_ptr(ids.device))
    N.check(rc, "fp_hybrid_row_limits")
    return out


def paged_prefill(q: Tensor, pool_k: Tensor, pool_v: Tensor, page_table: Tensor, batch_idx: Tensor,
                  row_limit: Tensor, page_size: int, *, scale: float | None = None,
                  out: Tensor | None = None, lse: Tensor | None = None,
                  sinks: Tensor | None = None, workspace: Tensor | None | bool = None,
                  score_bound: float = 0.0, tile_order: tuple[Tensor, int] | None = None) -> tuple[Tensor, Tensor]:
    """Chunked-prefill attention over the paged cache.  q [1, Hq, Lq, D]; row r sees keys
    0..row_limit[r]-1 of sequence batch_idx[r]; returns out like q, lse [1, Hq, Lq].
    `sinks` [Hq] float32 gates the output as in `paged_decode`.  `workspace`: a uint8 tensor of
    `prefill_workspace_bytes(...)` bytes lets a launch too small for the GPU be cut along the keys as
    well; None allocates one when the shape calls for it, False runs without.  `score_bound` > 0 is the
    caller's guarantee that |scale * q.k| never exceeds it (sqrt(D) for the model's normalised q and k): the
    bf16 kernel then runs its softmax without a running maximum.  `tile_order`: what `prefill_tile_order` returned
    for this step (order tensor, rows per tile): the launch's workgroups then run from the longest key range to
    the shortest; same results, faster where several small workgroups share a CU (head_dim 64)."""
    N.require_cuda(q, pool_k, pool_v, page_table, batch_idx, row_limit, out, lse)
    one, Hq, Lq, D = q.shape
    if one != 1:
        raise RuntimeError("paged_prefill takes the packed layout [1, Hq, Lq, D]")
    Hc, n_slots, Dp = pool_k.shape
    if Dp != D or pool_k.dtype != q.dtype or pool_v.dtype != q.dtype:
        raise RuntimeError("q / pool shape or dtype mismatch")
    q = _rows(q)
    if not batch_idx.is_contiguous():
        batch_idx = batch_idx.contiguous()
    if not row_limit.is_contiguous():
        row_limit = row_limit.contiguous()
    if batch_idx.dtype != torch.int64 or row_limit.dtype != torch.int32:
        raise RuntimeError("batch_idx must be int64 and row_limit int32")
    if batch_idx.numel() != Lq or row_limit.numel() != Lq:
        raise RuntimeError("batch_idx and row_limit need one entry per query row")
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if out is None:
        out = torch.empty_like(q)
    if lse is None:
        lse = torch.empty((1, Hq, Lq), dtype=torch.float32, device=q.device)
    if out.stride(3) != 1 or not lse.is_contiguous():
        raise RuntimeError("out rows must be dense and lse contiguous")
    if workspace is None:
        need = prefill_workspace_bytes(Lq, Hq, Hc, D, q.dtype)
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device) if need else False
    ws_ptr, ws_bytes = None, 0
    if workspace is not False:
        N.require_cuda(workspace)
        if workspace.dtype != torch.uint8 or not workspace.is_contiguous():
            raise RuntimeError("workspace must be a contiguous uint8 tensor")
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel()
    order_ptr, order_rows = None, 0
    if tile_order is not None:
        order, order_rows = tile_order
        N.require_cuda(order)
        if order.dtype != torch.int32 or not order.is_contiguous() or order.numel() != -(-Lq // order_rows):
            raise RuntimeError("tile_order must be what prefill_tile_order returned for this step: int32, one entry per "
                               f"tile of {order_rows} rows")
        order_ptr = order.data_ptr()
    rc = N.lib().fp_paged_prefill(
        q.data_ptr(), q.stride(2), q.stride(1), pool_k.data_ptr(), pool_v.data_ptr(),
        page_table.data_ptr(), page_table.stride(0), batch_idx.data_ptr(),
        row_limit.data_ptr(), out.data_ptr(), out.stride(2), out.stride(1), lse.data_ptr(),
        _sinks_ptr(sinks, Hq, q.device), Lq, Hq, Hc, D, page_size, page_table.shape[1], page_table.shape[0], n_slots,
        scale, float(score_bound), N.dtype_code(q.dtype), ws_ptr, ws_bytes, order_ptr, order_rows, N.stream_ptr(q.device))
    N.check(rc, "fp_paged_prefill")
    return out, lse


def prefill_tile_rows(Lq: int, Hq: int, Hc: int, D: int, dtype: torch.dtype, workspace_bytes: int = 0) -> int:
    """Rows per query tile of the launch `paged_prefill` makes for this shape with a workspace of this size
    (0: the launch takes no tile order)."""
    n = int(N.lib().fp_paged_prefill_tile_rows(Lq, Hq, Hc, D, N.dtype_code(dtype), workspace_bytes))
    N.check(n, "fp_paged_prefill_tile_rows")
    return n


def prefill_tile_order(batch_idx: Tensor, row_limit: Tensor, tile_rows: int) -> tuple[Tensor, int]:
    """The query tiles of a prefill step (tiles of `tile_rows` rows, `prefill_tile_rows`) by decreasing key range,
    as `(order, tile_rows)` for `paged_prefill(tile_order=)`.  Once per step: every layer's launch takes the same."""
    N.require_cuda(batch_idx, row_limit)
    batch_idx, row_limit = batch_idx.reshape(-1), row_limit.reshape(-1)
    if batch_idx.dtype != torch.int64 or row_limit.dtype != torch.int32 or batch_idx.numel() != row_limit.numel():
        raise RuntimeError("batch_idx must be int64 and row_limit int32, one entry per query row each")
    batch_idx, row_limit = batch_idx.contiguous(), row_limit.contiguous()
    Lq = row_limit.numel()
    order = torch.empty(-(-Lq // tile_rows) if tile_rows > 0 else 0, dtype=torch.int32, device=row_limit.device)
    rc = N.lib().fp_paged_prefill_tile_order(batch_idx.data_ptr(), row_limit.data_ptr(), Lq, tile_rows, order.data_ptr(),
                                             N.stream_ptr(row_limit.device))
    N.check(rc, "fp_paged_prefill_tile_order")
    return order, tile_rows


def prefill_workspace_bytes(Lq: int, Hq: int, Hc: int, D: int, dtype: torch.dtype) -> int:
    """Bytes of workspace with which `paged_prefill` cuts a launch of this shape along the keys as finely as
    it would like to on the current device (0: it would not cut it)."""
    n = int(N.lib().fp_paged_prefill_workspace_bytes(Lq, Hq, Hc, D, N.dtype_code(dtype)))
    N.check(n, "fp_paged_prefill_workspace_bytes")
    return n
