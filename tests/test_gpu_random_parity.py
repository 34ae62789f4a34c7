"""GPU parity on seeded random configurations: page size (powers of two and not), head grouping,
head_dim, dtype, context lengths, image spans and paddings are drawn per seed; every result is
compared with the oracle (bit-exact for the copies, the usual tolerances for attention)."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, bits, f64, randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float16: (4e-3, 4e-3), torch.float32: (3e-5, 3e-5)}
SOI, EOI, IMG, TXT = 5, 6, 7, 9


def draw(seed, dtypes):
    rng = np.random.default_rng(seed)
    P = int(rng.choice([1, 3, 8, 16, 24, 32, 64, 100, 128]))
    D = int(rng.choice([64, 128]))
    G = int(rng.choice([1, 2, 4, 8]))
    Hc = int(rng.choice([1, 2, 3]))
    dtype = dtypes[int(rng.integers(len(dtypes)))]
    return rng, P, D, G, Hc, dtype


@pytest.mark.parametrize("seed", range(12))
def test_decode_random(seed):
    rng, P, D, G, Hc, dtype = draw(seed, [torch.bfloat16, torch.float16, torch.float32])
    B = int(rng.integers(1, 7))
    lens = [int(x) for x in rng.integers(0, 700, B)]  # tokens cached before the step
    n_pages = sum(-(-(L + 1) // P) for L in lens) + 4
    st = PagedState(100 + seed, n_pages=n_pages, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    k1, v1 = randn(st.gen, (B, Hc, 1, D), dtype), randn(st.gen, (B, Hc, 1, D), dtype)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    pos = torch.tensor(lens, dtype=torch.int32)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pk, pv = st.pool_planes()
    max_ctx = -(-(max(lens) + 1) // 64) * 64
    split = int(rng.choice([64, 128, 256, 1024]))
    before = st.cache.kv_cache.clone()
    out, lse = ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), P, max_ctx,
                                split_tokens=split, k_new=k1.to(DEV), v_new=v1.to(DEV))
    # pool: the oracle's append on the previous contents, bit for bit
    want = before.cpu().clone()
    wv = want.view(torch.int16 if dtype != torch.float32 else torch.int32).numpy()
    O.append_decode(wv, 0, bits(k1), bits(v1), st.mirror.page_table, np.array(st.slots), pos.view(B, 1).numpy(), P)
    assert np.array_equal(bits(st.cache.kv_cache), wv)
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, pos.numpy(), P)
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse), el, atol=max(atol * 0.1, 2e-5), rtol=rtol)
    # gather returns exactly what was appended
    lens1 = torch.tensor([L + 1 for L in lens], device=DEV)
    got = ops.kv_gather(pk, st.cache.page_table, bidx, lens1, P, max(lens) + 1)
    ref = O.gather_pages(bits(pk), st.mirror.page_table, np.array(st.slots), np.array(lens) + 1, P, max(lens) + 1)
    assert np.array_equal(bits(got), ref)


@pytest.mark.parametrize("seed", range(10))
def test_prefill_random(seed):
    rng, P, D, G, Hc, dtype = draw(50 + seed, [torch.bfloat16, torch.float16, torch.float32])
    n_seq = int(rng.integers(1, 5))
    ids, bidx, pos, prefixes, slots = [], [], [], [], []
    total_pages = 0
    seqs = []
    for _ in range(n_seq):
        prefix = int(rng.integers(0, 300))   # already cached
        n_img = int(rng.integers(0, 120))
        n_txt = int(rng.integers(1, 150))
        chunk_ids = ([SOI] + [IMG] * n_img + [EOI] if n_img else []) + [TXT] * n_txt
        seqs.append((prefix, chunk_ids))
        total_pages += -(-(prefix + len(chunk_ids)) // P)
    st = PagedState(200 + seed, n_pages=total_pages + 4, page_size=P, max_batch=n_seq + 2, Hc=Hc, D=D, dtype=dtype)
    k_all, v_all = {}, {}
    for prefix, chunk_ids in seqs:
        b = st.add_sequence(prefix + len(chunk_ids))
        slots.append(b)
        pad = int(rng.integers(0, 4))
        ids += chunk_ids + [0] * pad
        bidx += [b] * len(chunk_ids) + [0] * pad
        pos += list(range(prefix, prefix + len(chunk_ids))) + [0] * pad
        prefixes.append(prefix)
    # the prefixes are plain text already in the pages
    for b, prefix in zip(slots, prefixes):
        if prefix:
            k = randn(st.gen, (1, Hc, prefix, D), dtype)
            v = randn(st.gen, (1, Hc, prefix, D), dtype)
            st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=torch.arange(prefix)[None].to(DEV),
                               batch_idx=torch.full((1, prefix), b).to(DEV))
    Lq = len(ids)
    ids_t, bidx_t, pos_t = (torch.tensor(x, dtype=torch.int64)[None].to(DEV) for x in (ids, bidx, pos))
    k = randn(st.gen, (1, Hc, Lq, D), dtype)
    v = randn(st.gen, (1, Hc, Lq, D), dtype)
    q = randn(st.gen, (1, Hc * G, Lq, D), dtype)
    mask = st.cache.create_prefill_blockmask(bidx_t, ids_t, SOI, EOI)
    st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pos_t, batch_idx=bidx_t)
    lim = mask.row_limit(pos_t)
    # the limits themselves: position + 1 outside a span, the span's end (in sequence coordinates) inside
    _, hi = O.row_windows(np.array(bidx), np.array(ids), SOI, EOI)
    want_lim = np.array(pos) + (hi - np.arange(Lq))
    assert np.array_equal(lim.cpu().numpy()[np.array(bidx) != 0], want_lim[np.array(bidx) != 0])
    pk, pv = st.pool_planes()
    out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx_t.view(-1), lim, P)
    eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, np.array(bidx), None,
                                       lim.cpu().numpy(), P)
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse), el, atol=max(atol * 0.1, 1e-4), rtol=rtol)


@pytest.mark.parametrize("seed", range(8))
def test_decode_random_large_launches(seed):
    """Many sequences and small splits, so that the launch has more workgroups than the GPU holds at once
    (the launch then takes the even cut over the flattened contexts): batch sizes that are no multiple
    of 64, empty and masked-out sequences, every page size and head grouping of `draw`; odd seeds with the
    step's plan."""
    rng, P, D, G, Hc, dtype = draw(200 + seed, [torch.bfloat16, torch.float16, torch.float32])
    Hc = int(rng.choice([4, 8]))
    B = int(rng.integers(90, 260))
    lens = [int(x) for x in rng.integers(0, 400, B)]
    lens[int(rng.integers(B))] = 0
    n_pages = sum(-(-(L + 1) // P) for L in lens) + 4
    st = PagedState(300 + seed, n_pages=n_pages, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    k1, v1 = randn(st.gen, (B, Hc, 1, D), dtype), randn(st.gen, (B, Hc, 1, D), dtype)
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    pos = torch.tensor(lens, dtype=torch.int32)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    masked = int(rng.integers(B))
    bidx[masked] = -1  # not a cache slot: out 0, lse -inf, nothing appended
    pk, pv = st.pool_planes()
    max_ctx = 448
    before = st.cache.kv_cache.clone()
    plan = None
    if seed % 2:  # every other configuration through the step's plan (fp_paged_decode_plan)
        plan = torch.zeros(ops.decode_plan_bytes(), dtype=torch.uint8, device=DEV)
        ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), P, max_ctx, split_tokens=64,
                         phase="plan", plan=plan)
        # (written where the launch is cut evenly; one-token pages with many sequences go split by split: untouched)
        assert int(plan.view(torch.int32)[1]) in (0, B)
    out, lse = ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), P, max_ctx,
                                split_tokens=64, k_new=k1.to(DEV), v_new=v1.to(DEV), plan=plan)
    keep = [i for i in range(B) if i != masked]
    want = before.cpu().clone()
    wv = want.view(torch.int16 if dtype != torch.float32 else torch.int32).numpy()
    O.append_decode(wv, 0, bits(k1)[keep], bits(v1)[keep], st.mirror.page_table, np.array(st.slots)[keep],
                    pos.view(B, 1).numpy()[keep], P)
    assert np.array_equal(bits(st.cache.kv_cache), wv)
    eo, el = O.decode_attention(f64(q)[keep], f64(pk), f64(pv), st.mirror.page_table, [st.slots[i] for i in keep],
                                pos.numpy()[keep], P)
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(out)[keep], eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse)[keep], el, atol=max(atol * 0.1, 2e-5), rtol=rtol)
    assert not f64(out)[masked].any() and np.isneginf(f64(lse)[masked]).all()
