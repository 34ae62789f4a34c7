"""Pins the oracle's attention: library routines (torch SDPA, scipy logsumexp),
closed forms, and invariances that any correct paged attention keeps."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F
from scipy.special import logsumexp

from oracle import paged_kv_oracle as O


def build(seed, n_seq=3, P=4, n_pages=20, Hc=2, G=2, D=8, max_len=15, perm=None):
    rng = np.random.default_rng(seed)
    a = O.PagedAllocator(n_pages, P, n_seq + 2)
    a.free_pages = (perm if perm is not None else rng.permutation(np.arange(1, n_pages))).tolist()
    lens = [int(x) for x in rng.integers(1, max_len + 1, size=n_seq)]
    slots, seqs = [], []
    pool = np.zeros((1, 2, 1, Hc, n_pages * P, D))
    for L in lens:
        b = a.allocate()
        a.reserve(b, L)
        k = rng.standard_normal((1, Hc, L, D))
        v = rng.standard_normal((1, Hc, L, D))
        O.append_prefill(pool, 0, k, v, a.page_table, np.full((1, L), b), np.arange(L)[None], P)
        slots.append(b)
        seqs.append((k[0], v[0]))
    q = rng.standard_normal((n_seq, Hc * G, 1, D))
    return a, pool, slots, lens, seqs, q


@pytest.mark.parametrize("seed", range(4))
@pytest.mark.parametrize("G", [1, 2, 4])
def test_decode_against_sdpa_and_logsumexp(seed, G):
    a, pool, slots, lens, seqs, q = build(seed, G=G)
    pos = np.array(lens) - 1
    out, lse = O.decode_attention(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, slots, pos, a.page_size)
    D = q.shape[-1]
    for b, (k, v) in enumerate(seqs):
        kk = torch.from_numpy(np.repeat(k, G, axis=0))[None]  # [1, Hq, L, D]
        vv = torch.from_numpy(np.repeat(v, G, axis=0))[None]
        ref = F.scaled_dot_product_attention(torch.from_numpy(q[b:b + 1]), kk, vv)
        np.testing.assert_allclose(out[b], ref[0].numpy(), rtol=1e-12, atol=1e-12)
        scores = np.einsum("hd,hld->hl", q[b, :, 0], np.repeat(k, G, axis=0)) / np.sqrt(D)
        np.testing.assert_allclose(lse[b, :, 0], logsumexp(scores, axis=1), rtol=1e-12, atol=1e-12)


def test_decode_single_key_closed_form():
    a, pool, slots, lens, seqs, q = build(11, n_seq=2, max_len=9)
    pos = np.zeros(2, dtype=np.int64)  # only position 0 visible
    out, lse = O.decode_attention(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, slots, pos, a.page_size)
    for b, (k, v) in enumerate(seqs):
        for h in range(q.shape[1]):
            np.testing.assert_allclose(out[b, h, 0], v[h // 2, 0], rtol=1e-13)
            np.testing.assert_allclose(lse[b, h, 0], q[b, h, 0] @ k[h // 2, 0] / np.sqrt(q.shape[-1]), rtol=1e-13)


def test_decode_equal_keys_gives_mean_of_values():
    a, pool, slots, lens, seqs, q = build(12, n_seq=1, max_len=12)
    L = lens[0]
    b = slots[0]
    t = np.arange(L)
    sl = a.page_table[b, t // a.page_size] * a.page_size + t % a.page_size
    pool[0, 0, 0][:, sl, :] = 0.37  # all keys equal
    out, lse = O.decode_attention(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, slots, [L - 1], a.page_size)
    np.testing.assert_allclose(out[0, 0, 0], seqs[0][1][0].mean(axis=0), rtol=1e-12)
    s = 0.37 * q[0, 0, 0].sum() / np.sqrt(q.shape[-1])
    np.testing.assert_allclose(lse[0, 0, 0], s + np.log(L), rtol=1e-12)


def test_decode_no_visible_key():
    a, pool, slots, lens, seqs, q = build(13, n_seq=2)
    out, lse = O.decode_attention(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, slots, [-1, lens[1] - 1], a.page_size)
    assert not out[0].any() and np.all(np.isneginf(lse[0]))
    assert np.all(np.isfinite(lse[1]))


def test_decode_is_invariant_to_the_page_permutation():
    n_pages = 20
    r1 = build(14, perm=np.arange(1, n_pages))
    r2 = build(14, perm=np.arange(1, n_pages)[::-1].copy())
    assert not np.array_equal(r1[0].page_table, r2[0].page_table)
    o1 = O.decode_attention(r1[5], r1[1][0, 0, 0], r1[1][0, 1, 0], r1[0].page_table, r1[2], np.array(r1[3]) - 1, 4)
    o2 = O.decode_attention(r2[5], r2[1][0, 0, 0], r2[1][0, 1, 0], r2[0].page_table, r2[2], np.array(r2[3]) - 1, 4)
    np.testing.assert_array_equal(o1[0], o2[0])
    np.testing.assert_array_equal(o1[1], o2[1])


@pytest.mark.parametrize("seed", range(3))
def test_masked_attention_dense_against_sdpa(seed):
    rng = np.random.default_rng(seed)
    Hq, Hc, Lq, Lk, D = 4, 2, 9, 13, 8
    q = rng.standard_normal((Hq, Lq, D))
    k = rng.standard_normal((Hc, Lk, D))
    v = rng.standard_normal((Hc, Lk, D))
    mask = rng.random((Lq, Lk)) < 0.6
    mask[:, 0] = True
    mask[4] = False  # one fully masked row
    out, lse = O.masked_attention_dense(q, k, v, mask)
    kk = torch.from_numpy(np.repeat(k, 2, axis=0))
    vv = torch.from_numpy(np.repeat(v, 2, axis=0))
    ok = [r for r in range(Lq) if r != 4]
    ref = F.scaled_dot_product_attention(torch.from_numpy(q)[:, ok], kk, vv, attn_mask=torch.from_numpy(mask)[ok])
    np.testing.assert_allclose(out[:, ok], ref.numpy(), rtol=1e-12, atol=1e-12)
    assert not out[:, 4].any() and np.all(np.isneginf(lse[:, 4]))
    s = np.einsum("hqd,hkd->hqk", q, np.repeat(k, 2, axis=0)) / np.sqrt(D)
    s = np.where(mask[None], s, -np.inf)
    np.testing.assert_allclose(lse[:, ok], logsumexp(s[:, ok], axis=2), rtol=1e-12)


@pytest.mark.parametrize("seed", range(3))
def test_paged_prefill_rows_equal_full_sequence_rows(seed):
    """A chunk attending over the paged prefix gives the rows of the whole-sequence result."""
    from tests.test_oracle_masks import EOI, SOI, packed_case

    rng = np.random.default_rng(seed)
    layout = [(1, [("t", 2), ("i", 7), ("t", 9)]), (2, [("i", 4), ("t", 6)])]
    ids, bidx, pos, spans = packed_case(layout)
    L = len(ids)
    Hq, Hc, D, P = 4, 2, 8, 4
    a = O.PagedAllocator(24, P, 4)
    a.free_pages = rng.permutation(np.arange(1, 24)).tolist()
    for slot in (1, 2):
        assert a.allocate() == slot
        a.reserve(slot, int((bidx == slot).sum()))
    q = rng.standard_normal((1, Hq, L, D))
    k = rng.standard_normal((1, Hc, L, D))
    v = rng.standard_normal((1, Hc, L, D))
    pool = np.zeros((1, 2, 1, Hc, 24 * P, D))
    O.append_prefill(pool, 0, k, v, a.page_table, bidx[None], pos[None], P)
    full, full_lse = O.prefill_attention_packed(q, k, v, bidx[None], ids[None], SOI, EOI)

    lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
    limit = pos + (hi - np.arange(L))
    real = bidx != 0
    # whole sequences at once
    out, lse = O.prefill_attention_paged(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, bidx, pos, limit, P)
    np.testing.assert_allclose(out[0][:, real], full[0][:, real], rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(lse[0][:, real], full_lse[0][:, real], rtol=1e-11)
    assert not out[0][:, ~real].any()
    # a chunk: the last 5 rows of sequence 1, prefix already in pages
    rows = np.flatnonzero(bidx == 1)[-5:]
    out_c, lse_c = O.prefill_attention_paged(q[:, :, rows], pool[0, 0, 0], pool[0, 1, 0], a.page_table,
                                             bidx[rows], pos[rows], limit[rows], P)
    np.testing.assert_allclose(out_c[0], full[0][:, rows], rtol=1e-11, atol=1e-12)


def test_text_only_chunk_is_plain_causal_attention():
    rng = np.random.default_rng(5)
    L, Hq, D, P = 11, 2, 8, 4
    a = O.PagedAllocator(8, P, 3)
    b = a.allocate()
    a.reserve(b, L)
    k = rng.standard_normal((1, Hq, L, D))
    v = rng.standard_normal((1, Hq, L, D))
    q = rng.standard_normal((1, Hq, L, D))
    pool = np.zeros((1, 2, 1, Hq, 8 * P, D))
    O.append_prefill(pool, 0, k, v, a.page_table, np.full((1, L), b), np.arange(L)[None], P)
    out, _ = O.prefill_attention_paged(q, pool[0, 0, 0], pool[0, 1, 0], a.page_table, np.full(L, b),
                                       np.arange(L), np.arange(L) + 1, P)
    ref = F.scaled_dot_product_attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), is_causal=True)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-12, atol=1e-12)
