"""CPU oracle for the paged KV-cache path (TEST INFRASTRUCTURE, not product code).

A slow, plain numpy restatement of what the reference's paged KV-cache path
computes.  Only tests, the smoke check and the CPU-baseline leg of the
benchmark may import this module; the product package never does.

Every function cites the reference lines it restates (paths relative to the
reference checkout, `falcon_perception/...`).  The attention arithmetic lives
in a third-party dependency of the reference (torch `flex_attention`, pinned
`torch>=2.11.0`, lowered through triton 3.6.0); its published definition is
restated here in float64: softmax(Q K^T * scale) V with a natural-log LSE,
`scale = 1/sqrt(D)`, fully masked rows give out = 0 and lse = -inf.

How each function is pinned (tests/test_oracle_*.py):
  PagedAllocator          hand-traced known answers from the reference source +
                          invariants under seeded random alloc/erase traces
  decode_slots/prefill_slots, append_*   brute-force python loops on tiny inputs,
                          "all other slots untouched", clamp and wrap cases
  gather_pages            inverse of append (round trip is the identity)
  convert_block_ids       closed form + brute force over all entries
  physical_mask           brute force over every physical slot
  causal_block_structure  torch.create_block_mask (library routine) on CPU
  hybrid_mask_dense       independent per-pair python predicate written from
                          the token layout, and the dense formulation of
                          mlx/attention.py:66-82 read as a spec
  row_windows             brute force against hybrid_mask_dense
  decode_attention, prefill_attention   scipy logsumexp / torch SDPA (library
                          routines), L=1 closed form, equal-keys -> mean(V),
                          page-permutation invariance
  rms_norm_rows           torch F.rms_norm (library routine); unit rms of the result
  rotary_3d               complex multiplication through torch.view_as_complex (library);
                          zero angle = identity, quarter turn (a, b) -> (-b, a), pair norms kept
  pre_attention_tail      composition of the two + numpy repeat against torch.repeat_interleave
  round_to_dtype          torch's own casts (library routine), ties and specials
  sink_gate               torch.sigmoid (library routine); closed forms: sink -> -inf
                          leaves out unchanged, sink == lse halves it, lse = -inf zeroes it
The reference holds no tests, golden vectors or fixtures for this path, so
those mathematical pins are all there is; none of the functions is unpinned.
"""

from __future__ import annotations

import numpy as np


def _cdiv(x: int, m: int) -> int:
    # paged_attention.py:23-24
    return int((x + m - 1) // m)


class PagedAllocator:
    """Page/slot allocator state machine, paged_attention.py:39-182.

    Tables are numpy int64 mirrors of the reference's device tensors.
    """

    def __init__(self, n_pages: int, page_size: int, max_batch_size: int):
        self.n_pages = n_pages
        self.page_size = page_size
        self.max_batch_size = max_batch_size
        # :58-60
        self.page_table = -np.ones((max_batch_size, n_pages), dtype=np.int64)
        self.page_table[0, :] = 0
        self.page_table_cpu = [[] for _ in range(max_batch_size)]
        # :63-67
        self.capacity = [0 for _ in range(max_batch_size)]
        self.free_pages = list(reversed(range(1, n_pages)))
        self.free_batch_idx = list(reversed(range(1, max_batch_size)))
        # :70
        self.physical_to_logical = -np.ones((max_batch_size, n_pages), dtype=np.int64)

    @property
    def num_free_pages(self) -> int:  # :111-113
        return len(self.free_pages)

    def can_reserve(self, size: int, batch_idx_int: int | None = None) -> bool:  # :95-100
        if batch_idx_int is None:
            return self.num_free_pages * self.page_size >= size and len(self.free_batch_idx) > 0
        return self.reserve(batch_idx_int, size, dry_run=True)

    def allocate(self) -> int:  # :102-109
        b = self.free_batch_idx.pop()
        self.capacity[b] = 0
        self.physical_to_logical[b, :] = -1
        self.page_table[b, :] = -1
        return b

    def reserve(self, b: int, seq_len: int, dry_run: bool = False) -> bool:  # :115-164
        if seq_len <= self.capacity[b]:
            return True
        n = _cdiv(seq_len - self.capacity[b], self.page_size)
        ok = n <= self.num_free_pages
        if dry_run:
            return ok
        if not ok:
            raise RuntimeError(
                f"Cannot reserve {n} pages for a sequence of length {seq_len} "
                f"in batch {b}. Only {self.num_free_pages} pages available. "
                f"Current capacity is {self.capacity[b]} tokens."
            )
        start = self.capacity[b] // self.page_size
        end = start + n
        pages = self.free_pages[-n:]  # list order, :149
        self.page_table[b, start:end] = pages
        self.physical_to_logical[b, pages] = np.arange(start, end)
        self.page_table_cpu[b] += pages
        self.free_pages = self.free_pages[:-n]
        self.capacity[b] += n * self.page_size
        return True

    def erase(self, b: int) -> None:  # :166-182
        self.free_batch_idx.append(b)
        self.free_pages.extend(reversed(self.page_table_cpu[b]))
        self.page_table_cpu[b] = []
        self.page_table[b, :] = -1
        self.physical_to_logical[b, :] = -1
        self.capacity[b] = 0


# --------------------------------------------------------------------------
# slot mapping and append
# --------------------------------------------------------------------------

def decode_slots(page_table, batch_idx, input_pos, page_size):
    """Flat slot per (b, s) for the decode append, paged_attention.py:212-224.

    page_table [maxB, Np] int64, batch_idx [B], input_pos [B, S].  Stale (-1)
    table entries are clamped to page 0 (:222).  Returns int64 [B*S], b-major.
    """
    page_table = np.asarray(page_table)
    batch_idx = np.asarray(batch_idx).astype(np.int64)
    input_pos = np.asarray(input_pos).astype(np.int64)
    blk = input_pos // page_size
    off = input_pos % page_size
    phys = np.take_along_axis(page_table[batch_idx], blk, axis=1)
    phys = np.maximum(phys, 0)
    return (phys * page_size + off).reshape(-1)


def prefill_slots(page_table, batch_idx, input_pos, page_size, n_slots):
    """Flat slot per packed token for the prefill append, paged_attention.py:387-389.

    batch_idx, input_pos [1, L].  No clamp; a negative result indexes from the
    end of the slot axis, as a negative index does in the reference's
    `kv_cache[..., idx, :] = val` (:390-391).
    """
    page_table = np.asarray(page_table)
    batch_idx = np.asarray(batch_idx).astype(np.int64)
    input_pos = np.asarray(input_pos).astype(np.int64)
    blk = input_pos // page_size
    off = input_pos % page_size
    idx = (page_table[batch_idx, blk] * page_size + off).reshape(-1)
    return np.where(idx < 0, idx + n_slots, idx)


def append_decode(pool, layer, k, v, page_table, batch_idx, input_pos, page_size):
    """Decode append, paged_attention.py:184-232.

    pool [L, 2, 1, H, N, D] is modified in place; k, v [B, H, S, D].
    Returns the views (pool[layer, 0], pool[layer, 1]) like :232.
    Rows are written in b-major order, so with duplicate slots the last row
    wins here; the reference leaves the order of duplicates unspecified.
    """
    B, H, S, D = k.shape
    assert pool.shape[3] == H and pool.shape[5] == D  # :205-207
    assert np.asarray(input_pos).shape == (B, S)  # :208
    assert np.asarray(batch_idx).shape == (B,)  # :209
    addr = decode_slots(page_table, batch_idx, input_pos, page_size)
    kk = np.ascontiguousarray(np.transpose(k, (1, 0, 2, 3))).reshape(H, B * S, D)  # :226
    vv = np.ascontiguousarray(np.transpose(v, (1, 0, 2, 3))).reshape(H, B * S, D)  # :227
    for t in range(B * S):
        pool[layer, 0, 0, :, addr[t], :] = kk[:, t, :]
        pool[layer, 1, 0, :, addr[t], :] = vv[:, t, :]
    return pool[layer, 0], pool[layer, 1]


def append_prefill(pool, layer, k, v, page_table, batch_idx, input_pos, page_size):
    """Prefill append, paged_attention.py:364-393.  k, v [1, H, L, D]; returns (k, v)."""
    assert np.asarray(batch_idx).ndim == 2 and np.asarray(batch_idx).shape[0] == 1  # :381-382
    assert np.asarray(input_pos).ndim == 2  # :383
    n_slots = pool.shape[4]
    idx = prefill_slots(page_table, batch_idx, input_pos, page_size, n_slots)
    for t in range(idx.shape[0]):
        pool[layer, 0, 0, :, idx[t], :] = k[0, :, t, :]
        pool[layer, 1, 0, :, idx[t], :] = v[0, :, t, :]
    return k, v


def gather_pages(pool_kv, page_table, batch_idx, seq_lens, page_size, max_len=None):
    """Logical view of the cached sequences: the inverse of the appends.

    pool_kv [H, N, D] (one of pool[layer, 0, 0] / pool[layer, 1, 0]).
    out[b, h, t, :] = pool_kv[h, page_table[batch_idx[b], t // P] * P + t % P, :]
    for t < seq_lens[b]; zero beyond.  The reference performs this lookup
    implicitly through the converted block indices (paged_attention.py:279-284).
    """
    pool_kv = np.asarray(pool_kv)
    H, N, D = pool_kv.shape
    B = len(batch_idx)
    if max_len is None:
        max_len = int(max(seq_lens)) if B else 0
    out = np.zeros((B, H, max_len, D), dtype=pool_kv.dtype)
    for b in range(B):
        L = int(seq_lens[b])
        t = np.arange(L)
        slots = np.asarray(page_table)[int(batch_idx[b]), t // page_size] * page_size + t % page_size
        out[b, :, :L, :] = pool_kv[:, slots, :]
    return out


# --------------------------------------------------------------------------
# page indexing of block masks
# --------------------------------------------------------------------------

def convert_block_ids(page_table, batch_idx, kv_indices, n_pages):
    """Logical -> physical block ids, paged_attention.py:279-284.

    kv_indices [B, H, R, C] int32 -> int32 [B, H, R, n_pages]; columns >= C are 0.
    """
    page_table = np.asarray(page_table)
    kv_indices = np.asarray(kv_indices)
    B, H, R, C = kv_indices.shape
    out = np.zeros((B, H, R, n_pages), dtype=np.int32)
    rows = page_table[np.asarray(batch_idx).astype(np.int64)]  # [B, Np]
    flat = kv_indices.reshape(B, -1).astype(np.int64)
    out[..., :C] = np.take_along_axis(rows, flat, axis=1).reshape(kv_indices.shape).astype(np.int32)
    return out


def physical_mask(physical_to_logical, batch_idx, page_size, logical_mask_fn, b, q_idx, phys_kv):
    """Element predicate in physical slot space, paged_attention.py:303-333."""
    lb = np.asarray(physical_to_logical)[int(batch_idx[b]), phys_kv // page_size]
    valid = lb >= 0
    logical = max(lb * page_size + phys_kv % page_size, 0)
    return bool(valid and logical_mask_fn(b, q_idx, logical))


def causal_block_structure(n_blocks):
    """Block lists of a causal mask whose block size equals the page size.

    What `create_causal_blockmask` (paged_attention.py:335-341) yields through
    torch's create_block_mask: row i has the one partial block {i} and the full
    blocks 0..i-1; index rows list the present blocks ascending, then the absent
    ones ascending (stable descending argsort of the dense block row).
    Returns (kv_num_blocks, kv_indices, full_kv_num_blocks, full_kv_indices),
    shapes [n], [n, n], [n], [n, n], int32.
    """
    n = n_blocks
    kv_num = np.ones(n, dtype=np.int32)
    full_num = np.arange(n, dtype=np.int32)
    kv_idx = np.zeros((n, n), dtype=np.int32)
    full_idx = np.zeros((n, n), dtype=np.int32)
    for i in range(n):
        kv_idx[i] = [i] + [j for j in range(n) if j != i]
        full_idx[i] = list(range(i)) + list(range(i, n))
    return kv_num, kv_idx, full_num, full_idx


# --------------------------------------------------------------------------
# hybrid mask
# --------------------------------------------------------------------------

def image_prefix_tables(input_ids, soi_id, eoi_id):
    """img_mask and img_indices of attention.py:79-88 for one packed row of ids."""
    ids = np.asarray(input_ids).reshape(-1)
    acc_soi = np.cumsum(ids == soi_id)
    acc_eoi = np.cumsum(ids == eoi_id)
    img_mask = (acc_soi - acc_eoi) > 0
    img_indices = acc_soi * img_mask
    return img_mask, img_indices


def hybrid_mask_dense(batch_idx, input_ids, soi_id, eoi_id):
    """Dense [L, L] bool prefill mask, paged_attention.py:343-362 + attention.py:75-96.

    allowed(q, kv) = image_prefix(q, kv) OR (q >= kv AND docs[q] == docs[kv]).
    """
    docs = np.asarray(batch_idx).reshape(-1)
    img_mask, img_idx = image_prefix_tables(input_ids, soi_id, eoi_id)
    L = docs.shape[0]
    q = np.arange(L)[:, None]
    kv = np.arange(L)[None, :]
    image_prefix = (img_mask[:, None] & img_mask[None, :]) & (img_idx[:, None] == img_idx[None, :])
    doc_causal = (q >= kv) & (docs[:, None] == docs[None, :])
    return image_prefix | doc_causal


def row_windows(batch_idx, input_ids, soi_id, eoi_id):
    """Per-row key window of the hybrid mask in packed coordinates.

    Within one document the allowed set of row q is the interval
    [doc_start(q), hi(q)) with hi(q) = max(q + 1, e(q)), e(q) = end of q's image
    span (or 0 outside a span).  Valid when every image span lies inside one
    document, which is what the engine packs (paged_inference.py:637-672).
    Returns (doc_start[L], hi[L]) int64.
    """
    docs = np.asarray(batch_idx).reshape(-1)
    img_mask, img_idx = image_prefix_tables(input_ids, soi_id, eoi_id)
    L = docs.shape[0]
    doc_start = np.zeros(L, dtype=np.int64)
    hi = np.zeros(L, dtype=np.int64)
    for q in range(L):
        s = q
        while s > 0 and docs[s - 1] == docs[q]:
            s -= 1
        doc_start[q] = s
        e = 0
        if img_mask[q]:
            e = q + 1
            while e < L and img_mask[e] and img_idx[e] == img_idx[q]:
                e += 1
        hi[q] = max(q + 1, e)
    return doc_start, hi


def chunk_row_limits(batch_idx, input_ids, soi_id, eoi_id, open_slots=()):
    """Row limits of a packed row of CHUNKS, with the conditions under which one limit per row is the mask.

    The reference prefills whole sequences (paged_inference.py:637-672), so its mask (attention.py:75-96,
    paged_attention.py:350-361) never meets a chunk that starts or ends inside an image span.  Per sequence
    the mask is allowed(q, kv) = kv <= q OR (q and kv inside one span [soi, eoi)); for a chunk whose slot
    is in `open_slots` the span was opened by an earlier chunk, so the rows before the chunk's first eoi
    are inside it.  Walks every document run (stretch of equal batch_idx) with its own open/closed state.

    Returns (hi[L] packed index one past the last visible key, status): status bit 0 = an eoi met with no
    span open, bit 1 = a span still open at the end of a run (document change or end of the row).
    """
    docs = np.asarray(batch_idx).reshape(-1)
    ids = np.asarray(input_ids).reshape(-1)
    L = docs.shape[0]
    hi = np.arange(1, L + 1, dtype=np.int64)
    status = 0
    k = 0
    while k < L:
        end = k
        while end < L and docs[end] == docs[k]:
            end += 1
        depth = 1 if int(docs[k]) in set(int(s) for s in open_slots) else 0
        start = k if depth else None  # first row of the span that is open now
        for t in range(k, end):
            if ids[t] == soi_id:
                if depth > 0 and start is not None:  # a soi inside an open span starts a new span id
                    hi[start:t] = np.maximum(hi[start:t], t)
                depth += 1
                start = t
            elif ids[t] == eoi_id:
                if depth <= 0:
                    status |= 1
                depth -= 1
                if depth <= 0 and start is not None:
                    hi[start:t] = np.maximum(hi[start:t], t)
                    start = None
        if depth > 0:
            status |= 2
        k = end
    return hi, status


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------

def _softmax_av(scores, vals):
    """scores [L] float64 (may be empty), vals [L, D] -> (out [D], lse)."""
    if scores.shape[0] == 0:
        return np.zeros(vals.shape[1], dtype=np.float64), -np.inf
    m = scores.max()
    e = np.exp(scores - m)
    s = e.sum()
    return (e[:, None] * vals).sum(axis=0) / s, m + np.log(s)


def decode_attention(q, pool_k, pool_v, page_table, batch_idx, input_pos, page_size, scale=None):
    """Single-query paged attention, float64.

    q [B, Hq, 1, D]; pool_k, pool_v [Hc, N, D] with Hq % Hc == 0; query head h
    reads cache head h // (Hq // Hc).  Sequence b sees logical positions
    0..input_pos[b] (the engine's mask `q + off[b] >= kv`,
    paged_inference.py:797-801) at slots page_table[batch_idx[b], t // P] * P + t % P.
    Returns out [B, Hq, 1, D] float64 and lse [B, Hq, 1] float64 (natural log;
    torch/nn/attention/flex_attention.py:1575-1598), scale 1/sqrt(D) (:1543-1544).
    A negative input_pos means no visible key: out 0, lse -inf
    (torch/_higher_order_ops/flex_attention.py:250-258).
    """
    q = np.asarray(q, dtype=np.float64)
    B, Hq, _, D = q.shape
    Hc = pool_k.shape[0]
    G = Hq // Hc
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.zeros((B, Hq, 1, D), dtype=np.float64)
    lse = np.full((B, Hq, 1), -np.inf, dtype=np.float64)
    pt = np.asarray(page_table)
    for b in range(B):
        L = int(np.asarray(input_pos).reshape(-1)[b]) + 1
        if L <= 0:
            continue
        t = np.arange(L)
        slots = pt[int(batch_idx[b]), t // page_size] * page_size + t % page_size
        for h in range(Hq):
            g = h // G
            K = np.asarray(pool_k[g][slots], dtype=np.float64)
            V = np.asarray(pool_v[g][slots], dtype=np.float64)
            s = (K @ q[b, h, 0]) * scale
            out[b, h, 0], lse[b, h, 0] = _softmax_av(s, V)
    return out, lse


def masked_attention_dense(q, k, v, mask, scale=None):
    """Dense masked attention, float64.  q [Hq, Lq, D], k, v [Hc, Lk, D], mask [Lq, Lk].

    Restates torch/_higher_order_ops/flex_attention.py:202-268 (math_attention)
    without its cast of P to the query dtype.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    Hq, Lq, D = q.shape
    G = Hq // k.shape[0]
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.zeros((Hq, Lq, v.shape[2]), dtype=np.float64)
    lse = np.full((Hq, Lq), -np.inf, dtype=np.float64)
    for h in range(Hq):
        s = (q[h] @ k[h // G].T) * scale
        s = np.where(mask, s, -np.inf)
        m = s.max(axis=1)
        ok = np.isfinite(m)
        msafe = np.where(ok, m, 0.0)
        e = np.exp(s - msafe[:, None])
        den = e.sum(axis=1)
        o = e @ v[h // G]
        out[h] = np.where(ok[:, None], o / np.where(ok, den, 1.0)[:, None], 0.0)
        lse[h] = np.where(ok, msafe + np.log(np.where(ok, den, 1.0)), -np.inf)
    return out, lse


def prefill_attention_packed(q, k, v, batch_idx, input_ids, soi_id, eoi_id, scale=None):
    """The reference's own prefill: attention over the packed fresh K/V under the
    hybrid mask (paged_attention.py:393, model.py:156-162).  q [1,Hq,L,D], k, v [1,Hc,L,D].
    """
    mask = hybrid_mask_dense(batch_idx, input_ids, soi_id, eoi_id)
    out, lse = masked_attention_dense(q[0], k[0], v[0], mask, scale)
    return out[None], lse[None]


def prefill_attention_paged(q, pool_k, pool_v, page_table, batch_idx, input_pos, row_limit,
                            page_size, scale=None):
    """Chunked prefill over the paged cache, float64.

    q [1, Hq, Lq, D] packed query rows; row r belongs to cache slot
    batch_idx[r] (its position input_pos[r] enters only through row_limit and may be
    None) and sees logical keys 0 .. row_limit[r]-1 of its own sequence (row_limit = max(pos + 1, image-span
    end): bidirectional inside the image span, causal elsewhere,
    attention.py:75-96), read from pages.  Rows with batch_idx 0 are padding:
    out 0, lse -inf.
    """
    q = np.asarray(q, dtype=np.float64)
    _, Hq, Lq, D = q.shape
    Hc = pool_k.shape[0]
    G = Hq // Hc
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.zeros((1, Hq, Lq, D), dtype=np.float64)
    lse = np.full((1, Hq, Lq), -np.inf, dtype=np.float64)
    bi = np.asarray(batch_idx).reshape(-1)
    lim = np.asarray(row_limit).reshape(-1)
    pt = np.asarray(page_table)
    cache = {}
    for r in range(Lq):
        b = int(bi[r])
        n = int(lim[r])
        if b == 0 or n <= 0:
            continue
        for h in range(Hq):
            g = h // G
            key = (b, g)
            if key not in cache or cache[key][0].shape[0] < n:
                nmax = int(lim[bi == b].max())
                tt = np.arange(nmax)
                ss = pt[b, tt // page_size] * page_size + tt % page_size
                cache[key] = (np.asarray(pool_k[g][ss], dtype=np.float64),
                              np.asarray(pool_v[g][ss], dtype=np.float64))
            K, V = cache[key]
            s = (K[:n] @ q[0, h, r]) * scale
            out[0, h, r], lse[0, h, r] = _softmax_av(s, V[:n])
    return out, lse


# --------------------------------------------------------------------------
# post-attention sink gate
# --------------------------------------------------------------------------
def round_to_dtype(x, dtype: str):
    """Value of float32 `x` after a round-to-nearest-even cast to `dtype` ("f32", "bf16", "f16") and back."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == "f32":
        return x.copy()
    if dtype == "f16":
        with np.errstate(over="ignore"):
            return x.astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        flat = np.ascontiguousarray(x).reshape(-1)
        bits = flat.view(np.uint32).astype(np.uint64)
        rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
        out = rounded.view(np.float32).copy()
        out[np.isnan(flat)] = np.nan
        return out.reshape(x.shape)
    raise ValueError(dtype)


def sink_gate(out, lse, sinks, dtype: str):
    """Attention._post_attention up to the transpose (model.py:122-126).

    out [B, H, S, D] attention output as values of the model dtype, lse [B, H, S] float32,
    sinks [H].  `sink_scale = sigmoid(lse - sinks.view(1, -1, 1))` in float32 (:124-125);
    `(out * sink_scale.unsqueeze(-1)).to(out.dtype)` (:126): float32 product, rounded to `dtype`."""
    out = round_to_dtype(out, dtype)
    lse = np.asarray(lse, dtype=np.float32)
    sinks = np.asarray(sinks, dtype=np.float32).reshape(1, -1, 1)
    with np.errstate(over="ignore"):
        scale = (1.0 / (1.0 + np.exp(-(lse - sinks).astype(np.float64)))).astype(np.float32)
    return round_to_dtype(out * scale[..., None], dtype)


# --------------------------------------------------------------------------
# QK norm + 3D rotary embedding in front of the cache insert
# --------------------------------------------------------------------------
def rms_norm_rows(x, eps, dtype: str):
    """F.rms_norm(x, (D,)) without weight (model.py:110-111): x * rsqrt(mean(x^2, -1) + eps) in
    float32, returned as values of `dtype`.  The reference passes eps=None, for which torch takes the
    machine epsilon of the float32 computation type also for bf16/f16 inputs (pinned against
    torch.nn.functional.rms_norm: bit-identical with 2^-23, not with the epsilon of bf16)."""
    x = np.asarray(x, dtype=np.float32)
    ms = np.mean(x.astype(np.float64) ** 2, axis=-1, keepdims=True).astype(np.float32)
    rstd = (1.0 / np.sqrt(ms.astype(np.float64) + eps)).astype(np.float32)
    return round_to_dtype(x * rstd, dtype)


def rotary_3d(x, freqs_cis, freqs_cis_2d, dtype: str):
    """apply_3d_rotary_emb for one tensor (rope.py:88-108).  x [B, S, H, D] values of `dtype`;
    freqs_cis complex [B, S, D/4] (rope.py:31-46: pairs (2i, 2i+1) of the first half times
    freqs_cis[b, s, i], broadcast over heads); freqs_cis_2d complex [B, S, H, D/4] or None
    (rope.py:71-86: even/odd elements of the second half rotated by the per-head angle)."""
    x = np.asarray(x, dtype=np.float32)
    D = x.shape[-1]
    half = D // 2
    out = x.copy()

    def rotate(part, cis):  # part [..., half] float32, cis complex broadcastable to [..., half/2]
        re, im = part[..., 0::2], part[..., 1::2]
        c = np.real(cis).astype(np.float32)
        s_ = np.imag(cis).astype(np.float32)
        res = np.empty_like(part)
        res[..., 0::2] = re * c - im * s_
        res[..., 1::2] = re * s_ + im * c
        return res

    out[..., :half] = rotate(x[..., :half], np.asarray(freqs_cis)[:, :, None, :])
    if freqs_cis_2d is not None:
        out[..., half:] = rotate(x[..., half:], np.asarray(freqs_cis_2d))
    return round_to_dtype(out, dtype)


def pre_attention_tail(xq, xk, xv, freqs_cis, freqs_cis_2d, n_rep: int, dtype: str, eps: float):
    """model.py:110-119: QK norm, repeat_kv (model.py:74-83, repeat_interleave along heads),
    3D rotary embedding, permute to [B, H, S, D].  Returns (q, k, v) as float32 values of `dtype`."""
    q = rms_norm_rows(xq, eps, dtype)
    k = rms_norm_rows(xk, eps, dtype)
    k = np.repeat(k, n_rep, axis=2)
    v = np.repeat(round_to_dtype(xv, dtype), n_rep, axis=2)
    q = rotary_3d(q, freqs_cis, freqs_cis_2d, dtype)
    k = rotary_3d(k, freqs_cis, freqs_cis_2d, dtype)
    return q.transpose(0, 2, 1, 3), k.transpose(0, 2, 1, 3), v.transpose(0, 2, 1, 3)
