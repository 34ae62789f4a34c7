"""Pins the oracle's slot mapping, appends, gather and block-id conversion.

Checks are independent of the oracle's own formulas: scalar python index
arithmetic on plain lists, torch's advanced-index assignment and torch.gather
(library routines) on CPU, and the round trip gather(append(x)) == x.
"""

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as O


def make_state(seed, n_pages=16, P=4, max_b=6, n_seq=3, max_len=13):
    rng = np.random.default_rng(seed)
    a = O.PagedAllocator(n_pages, P, max_b)
    perm = rng.permutation(np.arange(1, n_pages)).tolist()
    a.free_pages = perm  # fragmented pool
    lens, slots = [], []
    for _ in range(n_seq):
        b = a.allocate()
        L = int(rng.integers(1, max_len + 1))
        a.reserve(b, L)
        lens.append(L)
        slots.append(b)
    return a, slots, lens, rng


def scalar_slot(a, b, pos, clamp):
    page = a.page_table.tolist()[b][pos // a.page_size]
    if clamp and page < 0:
        page = 0
    return page * a.page_size + pos % a.page_size


@pytest.mark.parametrize("seed", range(4))
def test_decode_append_bruteforce(seed):
    a, slots, lens, rng = make_state(seed)
    H, D, S, Lyr = 3, 5, 2, 2
    N = a.n_pages * a.page_size
    pool0 = rng.standard_normal((Lyr, 2, 1, H, N, D)).astype(np.float32)
    pool = pool0.copy()
    B = len(slots)
    batch_idx = np.array(slots, dtype=np.int64)
    # S consecutive positions ending at the last reserved token of each sequence
    input_pos = np.array([[min(L - 1, s) if L < S else L - S + s for s in range(S)] for L in lens], dtype=np.int32)
    k = rng.standard_normal((B, H, S, D)).astype(np.float32)
    v = rng.standard_normal((B, H, S, D)).astype(np.float32)
    layer = 1
    rk, rv = O.append_decode(pool, layer, k, v, a.page_table, batch_idx, input_pos, a.page_size)
    assert rk.shape == (1, H, N, D) and np.shares_memory(rk, pool)

    expect = pool0.copy()
    for b in range(B):
        for s in range(S):
            slot = scalar_slot(a, slots[b], int(input_pos[b, s]), clamp=True)
            for h in range(H):
                expect[layer, 0, 0, h, slot] = k[b, h, s]
                expect[layer, 1, 0, h, slot] = v[b, h, s]
    assert np.array_equal(pool, expect)  # written rows right, every other slot untouched
    assert np.array_equal(pool[0], pool0[0])  # other layer untouched

    # the same through torch's advanced-index assignment (what the reference executes)
    tp = torch.from_numpy(pool0.copy())
    addr = torch.from_numpy(O.decode_slots(a.page_table, batch_idx, input_pos, a.page_size))
    tk = torch.from_numpy(k).permute(1, 0, 2, 3).contiguous().view(1, H, B * S, D)
    tv = torch.from_numpy(v).permute(1, 0, 2, 3).contiguous().view(1, H, B * S, D)
    tp[layer, 0, :, :, addr, :] = tk
    tp[layer, 1, :, :, addr, :] = tv
    assert np.array_equal(tp.numpy(), pool)


def test_decode_append_clamps_unmapped_rows_to_page0():
    a, slots, lens, rng = make_state(7)
    free_slot = a.free_batch_idx[-1]  # never allocated: its table row is all -1
    batch_idx = np.array([free_slot, 0], dtype=np.int64)
    input_pos = np.array([[5], [9]], dtype=np.int32)
    got = O.decode_slots(a.page_table, batch_idx, input_pos, a.page_size)
    # -1 clamps to page 0; slot row 0 maps every block to page 0
    assert got.tolist() == [5 % a.page_size, 9 % a.page_size]


@pytest.mark.parametrize("seed", range(3))
def test_prefill_append_matches_torch_index_put(seed):
    a, slots, lens, rng = make_state(seed + 10)
    H, D = 2, 4
    N = a.n_pages * a.page_size
    bidx, pos = [], []
    for b, L in zip(slots, lens):
        bidx += [b] * L + [0] * ((-L) % 4)  # pad each sequence to a multiple of 4 with (0, 0) rows
        pos += list(range(L)) + [0] * ((-L) % 4)
    Lp = len(bidx)
    batch_idx = np.array([bidx], dtype=np.int64)
    input_pos = np.array([pos], dtype=np.int64)
    k = rng.standard_normal((1, H, Lp, D)).astype(np.float32)
    v = rng.standard_normal((1, H, Lp, D)).astype(np.float32)
    pool0 = rng.standard_normal((1, 2, 1, H, N, D)).astype(np.float32)
    pool = pool0.copy()
    rk, rv = O.append_prefill(pool, 0, k, v, a.page_table, batch_idx, input_pos, a.page_size)
    assert rk is k and rv is v  # the inputs come back (reference :393)

    idx = O.prefill_slots(a.page_table, batch_idx, input_pos, a.page_size, N)
    for t in range(Lp):
        assert idx[t] == scalar_slot(a, bidx[t], pos[t], clamp=False)
    real = np.array(bidx) != 0
    tp = torch.from_numpy(pool0.copy())
    tidx = torch.from_numpy(idx)
    tp[0, 0, :, :, tidx, :] = torch.from_numpy(k)
    tp[0, 1, :, :, tidx, :] = torch.from_numpy(v)
    # slot 0 (all padding rows collide there) is unspecified; everything else must agree
    assert np.array_equal(tp.numpy()[..., 1:, :], pool[..., 1:, :])
    assert set(idx[~real].tolist()) <= {0}
    untouched = np.setdiff1d(np.arange(N), idx)
    assert np.array_equal(pool[..., untouched, :], pool0[..., untouched, :])


def test_prefill_negative_slot_wraps_like_a_negative_index():
    a = O.PagedAllocator(4, 4, 3)
    b = a.allocate()  # nothing reserved: page_table[b] == -1
    idx = O.prefill_slots(a.page_table, np.array([[b]]), np.array([[2]]), 4, 16)
    assert idx.tolist() == [16 + (-1 * 4 + 2)]
    t = torch.zeros(16)
    t[torch.tensor([-1 * 4 + 2])] = 1.0  # torch resolves the negative index the same way
    assert t.nonzero().item() == idx[0]


@pytest.mark.parametrize("seed", range(4))
def test_gather_is_the_inverse_of_append(seed):
    a, slots, lens, rng = make_state(seed + 20, n_pages=24, n_seq=4, max_len=17)
    H, D = 3, 4
    N = a.n_pages * a.page_size
    pool = np.zeros((1, 2, 1, H, N, D), dtype=np.float32)
    seqs = []
    for b, L in zip(slots, lens):
        x = rng.standard_normal((1, H, L, D)).astype(np.float32)
        O.append_prefill(pool, 0, x, -x, a.page_table, np.full((1, L), b), np.arange(L)[None], a.page_size)
        seqs.append(x)
    Lmax = max(lens) + 2
    gk = O.gather_pages(pool[0, 0, 0], a.page_table, slots, lens, a.page_size, Lmax)
    gv = O.gather_pages(pool[0, 1, 0], a.page_table, slots, lens, a.page_size, Lmax)
    for i, (x, L) in enumerate(zip(seqs, lens)):
        assert np.array_equal(gk[i, :, :L], x[0])
        assert np.array_equal(gv[i, :, :L], -x[0])
        assert not gk[i, :, L:].any()


def test_convert_block_ids_closed_form():
    a, slots, lens, rng = make_state(3, n_pages=12)
    B, Hm, R, C = len(slots), 1, 2, 5
    kv_idx = rng.integers(0, a.n_pages, size=(B, Hm, R, C)).astype(np.int32)
    got = O.convert_block_ids(a.page_table, slots, kv_idx, a.n_pages)
    assert got.dtype == np.int32 and got.shape == (B, Hm, R, a.n_pages)
    pt = a.page_table.tolist()
    for b in range(B):
        for r in range(R):
            for c in range(a.n_pages):
                exp = pt[slots[b]][kv_idx[b, 0, r, c]] if c < C else 0
                assert got[b, 0, r, c] == exp
    # torch.gather, the routine the reference calls (:282)
    tg = torch.gather(torch.from_numpy(a.page_table)[torch.tensor(slots)], 1,
                      torch.from_numpy(kv_idx).view(B, -1).long()).view(B, Hm, R, C).int()
    assert np.array_equal(tg.numpy(), got[..., :C])


def test_physical_mask_bruteforce():
    a, slots, lens, rng = make_state(5, n_pages=10)
    P = a.page_size
    causal = lambda b, q, kv: q >= kv
    for bi, (b, L) in enumerate(zip(slots, lens)):
        q = L - 1
        inverse = {p: lb for lb, p in enumerate(a.page_table_cpu[b])}
        for phys in range(a.n_pages * P):
            page = phys // P
            exp = page in inverse and (inverse[page] * P + phys % P) <= q
            assert O.physical_mask(a.physical_to_logical, slots, P, causal, bi, q, phys) == exp
