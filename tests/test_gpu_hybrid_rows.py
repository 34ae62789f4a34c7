"""GPU parity: per-row key limits of the hybrid mask equal the oracle's dense mask rows."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV
from tests.test_oracle_masks import EOI, IMG, LAYOUTS, SOI, TXT, packed_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layout", LAYOUTS)
def test_row_limits_on_engine_layouts(layout):
    ids, bidx, pos, spans = packed_case(layout)
    got = ops.hybrid_row_limits(torch.from_numpy(ids)[None].to(DEV), SOI, EOI).cpu().numpy()
    lo, hi = O.row_windows(bidx[None], ids[None], SOI, EOI)
    assert got.dtype == np.int32 and np.array_equal(got, hi)


@pytest.mark.parametrize("L", [1, 7, 1024, 1025, 5000, 65536])
def test_row_limits_on_random_delimiters(L):
    rng = np.random.default_rng(L)
    ids = rng.choice([SOI, EOI, IMG, TXT], size=L, p=[0.02, 0.02, 0.6, 0.36])
    got = ops.hybrid_row_limits(torch.from_numpy(ids).to(DEV), SOI, EOI).cpu().numpy()
    img, idx = O.image_prefix_tables(ids, SOI, EOI)
    # end of the run of equal (img, idx) that contains q, computed with numpy on the whole row
    key = np.where(img, idx, -1 - np.arange(L))  # non-image rows are runs of length one
    change = np.flatnonzero(np.diff(key) != 0) + 1
    ends = np.append(change, L)
    run_end = ends[np.searchsorted(ends, np.arange(L), side="right")]
    exp = np.where(img, run_end, np.arange(L) + 1)
    assert np.array_equal(got, exp)
    if L <= 5000:
        lo, hi = O.row_windows(np.ones((1, L), dtype=np.int64), ids[None], SOI, EOI)
        assert np.array_equal(got, hi)


def limits_with_status(ids, bidx, open_slots, max_batch=8):
    flags = torch.zeros(max_batch, dtype=torch.uint8)
    flags[list(open_slots)] = 1
    status = torch.full((1,), 77, dtype=torch.int32, device=DEV)  # the kernel writes, it does not accumulate
    got = ops.hybrid_row_limits(torch.from_numpy(ids).to(DEV), SOI, EOI, torch.from_numpy(bidx).to(DEV),
                                flags.to(DEV) if open_slots is not None else None, status)
    return got.cpu().numpy(), int(status.item())


@pytest.mark.parametrize("layout", LAYOUTS)
def test_every_cut_of_a_packed_row(layout):
    """The packed row cut in two at every index: limits and status of both pieces equal the oracle's
    (a piece that starts inside a span is declared open, or flagged when it is not)."""
    ids, bidx, pos, spans = packed_case(layout)
    L = len(ids)
    for p in range(1, L):
        head, hs = limits_with_status(ids[:p], bidx[:p], [])
        eh, es = O.chunk_row_limits(bidx[:p], ids[:p], SOI, EOI)
        assert hs == es, p
        if es == 0:
            assert np.array_equal(head, eh), p
        inside = [int(bidx[p])] if any(a < p <= e for a, e in spans) else []
        tail, ts = limits_with_status(ids[p:], bidx[p:], inside)
        et, es = O.chunk_row_limits(bidx[p:], ids[p:], SOI, EOI, open_slots=inside)
        assert ts == es == 0, p
        assert np.array_equal(tail, et), p
        if inside:
            assert limits_with_status(ids[p:], bidx[p:], [])[1] == O.chunk_row_limits(bidx[p:], ids[p:], SOI, EOI)[1] != 0


def test_status_on_long_rows():
    """Flags raised by threads far from thread 0: 5000 rows, the offending token near the end."""
    L = 5000
    ids = np.full(L, TXT)
    bidx = np.ones(L, dtype=np.int64)
    bidx[4000:] = 2
    assert limits_with_status(ids, bidx, [])[1] == 0
    ids[4500] = EOI
    assert limits_with_status(ids, bidx, [])[1] == 1
    got, status = limits_with_status(ids, bidx, [2])
    exp, es = O.chunk_row_limits(bidx, ids, SOI, EOI, open_slots=[2])
    assert status == es == 0 and np.array_equal(got, exp)
    assert (got[4000:4500] == 4500).all() and got[3999] == 4000
    ids[3990] = SOI  # open where the document changes
    assert limits_with_status(ids, bidx, [2])[1] == 2
    ids[4990] = SOI  # and where the row ends
    ids[3990] = TXT
    assert limits_with_status(ids, bidx, [2])[1] == 2


def test_status_of_a_span_open_across_a_document_boundary():
    """Where the kernel's status and the oracle's differ: a span left open by document 1 and an eoi in document 2.
    The kernel counts delimiters over the whole packed row, as the reference's mask does (attention.py:75-96), so
    the second document's eoi closes the first document's span and no balance ever drops below zero: status 2.
    The oracle walks every document with its own balance and also sees an eoi with no span open: status 3.  Bit 1
    is set by both, and bit 1 alone rejects the step."""
    ids = np.array([TXT] * 3 + [SOI] + [IMG] * 20 + [TXT] * 8 + [EOI] + [TXT] * 4)
    bidx = np.array([1] * 24 + [2] * 13)
    _, status = limits_with_status(ids, bidx, [])
    _, es = O.chunk_row_limits(bidx, ids, SOI, EOI)
    assert status == 2 and es == 3 and (status & es & 2)
