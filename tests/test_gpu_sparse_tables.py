"""GPU parity with a sparse page table: [max_batch, max blocks per sequence] instead of the
reference's dense [max_batch, n_pages] (paged_attention.py:58), no inverse table.  Page ids are then
larger than the table is wide; every kernel must give the bits it gives with the dense table."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, bits, f64, randn

pytestmark = pytest.mark.gpu


def build(cols):
    st = PagedState(41, n_pages=400, page_size=16, max_batch=6, Hc=2, D=128, dtype=torch.bfloat16,
                    max_blocks_per_seq=cols)
    for L in (500, 33, 512, 1):
        st.add_sequence(L)
    return st


def test_append_gather_decode_prefill_equal_the_dense_table_results():
    results = []
    for cols in (None, 32):  # 32 blocks x 16 tokens = 512 tokens per sequence; pool page ids run to 399
        st = build(cols)
        assert st.cache.page_table.shape == (6, 400 if cols is None else 32)
        assert (st.cache.physical_to_logical is None) == (cols is not None)
        assert int(st.cache.page_table.max()) > 32  # ids beyond the table width are ordinary pages
        st.prefill_random()
        pk, pv = st.pool_planes()
        bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
        lens = torch.tensor(st.lens, device=DEV)
        gathered = ops.kv_gather(pk, st.cache.page_table, bidx, lens, st.P, 512)
        q = randn(st.gen, (4, 4, 1, 128), torch.bfloat16).to(DEV)
        pos = (lens - 1).to(torch.int32)
        out, lse = ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, 512, split_tokens=128)
        qp = randn(st.gen, (1, 4, 1045, 128), torch.bfloat16).to(DEV)
        rows_b = torch.cat([torch.full((L,), b) for b, L in zip(st.slots[:3], st.lens[:3])]).to(DEV)
        lim = torch.cat([torch.arange(1, L + 1) for L in st.lens[:3]]).to(torch.int32).to(DEV)
        po, pl = ops.paged_prefill(qp[:, :, : rows_b.shape[0]], pk, pv, st.cache.page_table, rows_b, lim, st.P)
        results.append((st, st.cache.kv_cache.clone(), gathered, out, lse, po, pl))
    dense, sparse = results
    for a, b in zip(dense[1:], sparse[1:]):
        assert np.array_equal(bits(a), bits(b))
    # and the dense result is the oracle's (decode, as one anchor)
    st = dense[0]
    pk, pv = st.pool_planes()
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots,
                                np.array(st.lens) - 1, st.P)
    np.testing.assert_allclose(f64(sparse[3]), eo, atol=2e-2, rtol=1e-2)


def test_a_sequence_cannot_outgrow_the_table():
    st = build(32)
    b = st.slots[0]
    assert st.cache.reserve(b, None, 513, dry_run=True) is False
    with pytest.raises(RuntimeError, match="32 blocks"):
        st.cache.reserve(b, None, 513)
    with pytest.raises(RuntimeError, match="physical_to_logical"):
        st.cache.get_logical_kv_idx(torch.zeros(1, dtype=torch.long, device=DEV), torch.zeros(1, dtype=torch.long, device=DEV),
                                    torch.tensor([b], device=DEV))
    # erase and reuse keep working without the inverse table
    st.cache.erase(b)
    nb = st.cache.allocate()
    st.cache.reserve(nb, None, 100)
    assert st.cache.capacity[nb] == 112 and (st.cache.page_table[nb, :7] > 0).all() and (st.cache.page_table[nb, 7:] == -1).all()
