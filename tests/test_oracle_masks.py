"""Pins the oracle's mask functions: causal block structure, hybrid mask, row windows."""

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import create_block_mask

from oracle import paged_kv_oracle as O

SOI, EOI, IMG, PAD, TXT = 101, 102, 103, 0, 7


@pytest.mark.parametrize("n", [1, 2, 5, 8])
def test_causal_block_structure_matches_torch(n):
    P = 4
    bm = create_block_mask(lambda b, h, q, kv: q >= kv, 1, None, n * P, n * P, device="cpu", BLOCK_SIZE=P)
    kv_num, kv_idx, full_num, full_idx = O.causal_block_structure(n)
    assert np.array_equal(bm.kv_num_blocks[0, 0].numpy(), kv_num)
    assert np.array_equal(bm.kv_indices[0, 0].numpy(), kv_idx)
    if n > 1:
        assert np.array_equal(bm.full_kv_num_blocks[0, 0].numpy(), full_num)
        # only the first full_num[i] entries of a row are ever read
        for i in range(n):
            assert np.array_equal(bm.full_kv_indices[0, 0, i, :i].numpy(), full_idx[i, :i])


def packed_case(layout):
    """layout: list of (slot, [segments]); a segment is ('t', n) text or ('i', n) an image
    block cls + 4 reg + n img + eoi (reference data.py:513-522).  Each sequence is padded
    to a multiple of 8 with (slot 0, PAD) rows.  Returns ids, batch_idx, pos and, built
    from the construction itself, the list of image spans [a, e) in packed coordinates."""
    ids, bidx, pos, spans = [], [], [], []
    for slot, segs in layout:
        start = len(ids)
        for kind, n in segs:
            if kind == "t":
                ids += [TXT] * n
            else:
                a = len(ids)
                ids += [SOI] + [IMG + 1] * 4 + [IMG] * n + [EOI]
                spans.append((a, len(ids) - 1))  # eoi itself is outside the bidirectional span
        L = len(ids) - start
        bidx += [slot] * L
        pos += list(range(L))
        gap = (-L) % 8
        ids += [PAD] * gap
        bidx += [0] * gap
        pos += [0] * gap
    return np.array(ids), np.array(bidx), np.array(pos), spans


def expected_pair(q, kv, bidx, spans):
    """The mask written down independently: same document and causal, or both inside one image span."""
    if bidx[q] == bidx[kv] and kv <= q:
        return True
    return any(a <= q < e and a <= kv < e for a, e in spans)


LAYOUTS = [
    [(1, [("t", 3), ("i", 6), ("t", 5)])],
    [(2, [("i", 9), ("t", 4)]), (1, [("t", 11)])],
    [(3, [("t", 2), ("i", 3), ("t", 2), ("i", 5), ("t", 1)]), (5, [("i", 2)])],
    [(1, [("t", 8)]), (2, [("t", 16)])],
]


@pytest.mark.parametrize("layout", LAYOUTS)
def test_hybrid_mask_against_construction(layout):
    ids, bidx, pos, spans = packed_case(layout)
    got = O.hybrid_mask_dense(bidx[None], ids[None], SOI, EOI)
    L = len(ids)
    for q in range(L):
        for kv in range(L):
            assert got[q, kv] == expected_pair(q, kv, bidx, spans), (q, kv)


@pytest.mark.parametrize("layout", LAYOUTS)
def test_hybrid_mask_against_dense_formulation(layout):
    """The dense composition spelled out in the reference's MLX twin (mlx/attention.py:66-82)."""
    ids, bidx, pos, spans = packed_case(layout)
    soi = (ids == SOI).astype(np.int64)
    eoi = (ids == EOI).astype(np.int64)
    acc_s, acc_e = np.cumsum(soi), np.cumsum(eoi)
    img = (acc_s - acc_e) > 0
    idx = acc_s * img
    image_prefix = img[:, None] & img[None, :] & (idx[:, None] == idx[None, :])
    L = len(ids)
    causal = np.arange(L)[:, None] >= np.arange(L)[None, :]
    doc = bidx[:, None] == bidx[None, :]
    assert np.array_equal(O.hybrid_mask_dense(bidx[None], ids[None], SOI, EOI), image_prefix | (causal & doc))


@pytest.mark.parametrize("layout", LAYOUTS)
def test_row_windows_equal_the_dense_rows(layout):
    ids, bidx, pos, spans = packed_case(layout)
    dense = O.hybrid_mask_dense(bidx[None], ids[None], SOI, EOI)
    lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
    for q in range(len(ids)):
        if bidx[q] == 0:
            continue  # padding rows of different gaps see each other; not an interval
        allowed = np.flatnonzero(dense[q])
        assert allowed.tolist() == list(range(lo[q], hi[q])), q


def test_irregular_delimiters_keep_spans_contiguous():
    """Whatever the soi/eoi pattern, the image-prefix set of a row is one contiguous run."""
    rng = np.random.default_rng(0)
    for _ in range(50):
        ids = rng.choice([SOI, EOI, IMG, TXT], size=40)
        bidx = np.ones(40, dtype=np.int64)
        img_mask, img_idx = O.image_prefix_tables(ids, SOI, EOI)
        for q in np.flatnonzero(img_mask):
            same = np.flatnonzero(img_mask & (img_idx == img_idx[q]))
            assert same.tolist() == list(range(same[0], same[-1] + 1))
            lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
            assert hi[q] == max(q + 1, same[-1] + 1)


# ---------------------------------------------------------------- chunks that cut an image span

@pytest.mark.parametrize("layout", LAYOUTS)
def test_chunk_row_limits_equal_row_windows_on_whole_sequences(layout):
    ids, bidx, pos, spans = packed_case(layout)
    lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
    got, status = O.chunk_row_limits(bidx[None], ids[None], SOI, EOI)
    assert status == 0
    real = bidx != 0
    assert np.array_equal(got[real], hi[real])


def test_chunk_row_limits_equal_row_windows_on_irregular_delimiters():
    rng = np.random.default_rng(1)
    clean = 0
    for _ in range(600):
        ids = rng.choice([SOI, EOI, IMG, TXT], size=16, p=[0.1, 0.1, 0.4, 0.4])
        bidx = np.ones(16, dtype=np.int64)
        got, status = O.chunk_row_limits(bidx[None], ids[None], SOI, EOI)
        opened = np.cumsum(ids == SOI) - np.cumsum(ids == EOI)
        assert bool(status & 1) == bool((opened < 0).any())
        assert bool(status & 2) == bool(opened[-1] > 0)
        if status == 0:
            clean += 1
            assert np.array_equal(got, O.row_windows(bidx[None], ids[None], SOI, EOI)[1])
    assert clean > 20


@pytest.mark.parametrize("segs", [
    [("t", 3), ("i", 6), ("t", 5)],
    [("i", 9), ("t", 4)],
    [("t", 2), ("i", 3), ("t", 2), ("i", 5), ("t", 1)],
])
def test_chunk_boundaries_inside_the_image_span(segs):
    """A sequence cut in two at every position: the second chunk's limits, with the span declared open
    when the cut falls inside one, are the rows of the whole-sequence mask; the first chunk is refused
    exactly when the cut falls inside a span (its rows would need keys that are not cached yet; a cut right
    in front of the eoi counts as inside, since nothing in the first chunk says that the span ends there)."""
    ids, bidx, pos, spans = packed_case([(3, segs)])
    n = int((bidx != 0).sum())
    ids, bidx = ids[:n], bidx[:n]
    dense = O.hybrid_mask_dense(bidx[None], ids[None], SOI, EOI)
    want = np.array([np.flatnonzero(dense[q])[-1] + 1 for q in range(n)])
    for q in range(n):  # one limit per row is the whole mask: the allowed keys of a row are 0 .. want - 1
        assert np.flatnonzero(dense[q]).tolist() == list(range(want[q]))
    for p in range(1, n):
        cut_inside = any(a < p <= e for a, e in spans)  # the soi lies before the cut, its eoi (index e) does not
        head, status = O.chunk_row_limits(bidx[None, :p], ids[None, :p], SOI, EOI)
        assert status == (2 if cut_inside else 0), p
        if not cut_inside:
            assert np.array_equal(head, want[:p])
        tail, status = O.chunk_row_limits(bidx[None, p:], ids[None, p:], SOI, EOI, open_slots=[3] if cut_inside else [])
        assert status == 0, p
        assert np.array_equal(tail + p, want[p:]), p
        if cut_inside:  # undeclared: the eoi closes nothing
            assert O.chunk_row_limits(bidx[None, p:], ids[None, p:], SOI, EOI)[1] & 1


def test_span_open_across_a_document_boundary_is_flagged():
    ids = np.array([TXT, SOI, IMG, IMG, TXT, TXT, EOI, TXT])
    bidx = np.array([1, 1, 1, 1, 2, 2, 2, 2])
    # the reference's global counts would let rows 1..3 see rows 4..5 of the other document
    dense = O.hybrid_mask_dense(bidx[None], ids[None], SOI, EOI)
    assert dense[2, 5]
    hi, status = O.chunk_row_limits(bidx[None], ids[None], SOI, EOI)
    assert status == 3  # open at the boundary, and document 2's eoi closes nothing of its own
