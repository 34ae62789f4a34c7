"""GPU parity: KV append, page gather and block-id conversion are bit-exact against the oracle."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, bits, check_tables_match, randn

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def oracle_pool(state, layers=1):
    c = state.cache
    return np.zeros(tuple(c.kv_cache.shape), dtype=bits(c.kv_cache[:0]).dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("D", [64, 128, 20])
def test_prefill_append_bit_exact(dtype, D):
    st = PagedState(1, n_pages=40, page_size=16, max_batch=6, Hc=3, D=D, dtype=dtype, n_layers=2)
    for L in (1, 16, 17, 100, 33):
        st.add_sequence(L)
    check_tables_match(st)
    k, v, bt, pt, rk, rv = st.prefill_random(layer=1, pad_to=8)
    assert rk.data_ptr() != st.cache.kv_cache.data_ptr()  # the fresh rows come back, not the pool
    ref = oracle_pool(st)
    O.append_prefill(ref, 1, bits(k), bits(v), st.mirror.page_table, bt.numpy(), pt.numpy(), st.P)
    got = bits(st.cache.kv_cache)
    assert np.array_equal(got[..., 1:, :], ref[..., 1:, :])  # slot 0 takes the colliding padding rows
    assert not got[0].any()  # layer 0 untouched


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("S", [1, 3])
def test_decode_append_bit_exact(dtype, S):
    st = PagedState(2, n_pages=64, page_size=64, max_batch=8, Hc=8, D=64, dtype=dtype)
    for L in (64, 200, 65, 512, 130):
        st.add_sequence(L)
    st.prefill_random()
    before = bits(st.cache.kv_cache).copy()
    B, H, D = len(st.slots), st.Hc, st.D
    # the model hands K/V over as a permuted [B, S, H, D] tensor (reference model.py:118-119)
    k = randn(st.gen, (B, S, H, D), dtype).permute(0, 2, 1, 3)
    v = randn(st.gen, (B, S, H, D), dtype).permute(0, 2, 1, 3)
    pos = torch.tensor([[L - S + s for s in range(S)] for L in st.lens], dtype=torch.int32)
    bidx = torch.tensor(st.slots, dtype=torch.int64)
    rk, rv = st.cache.insert_kv(0, k.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3),
                                v.to(DEV).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3),
                                input_pos=pos.to(DEV), batch_idx=bidx.to(DEV))
    # decode returns views of the whole pool of the layer
    assert rk.shape == (1, H, st.cache.n_pages * st.P, D)
    assert rk.data_ptr() == st.cache.kv_cache[0, 0].data_ptr() and rv.data_ptr() == st.cache.kv_cache[0, 1].data_ptr()
    ref = before.copy()
    O.append_decode(ref, 0, bits(k), bits(v), st.mirror.page_table, bidx.numpy(), pos.numpy(), st.P)
    assert np.array_equal(bits(st.cache.kv_cache), ref)


def test_decode_append_padding_rows_go_to_page0():
    dtype = torch.bfloat16
    st = PagedState(3, n_pages=32, page_size=16, max_batch=6, Hc=4, D=128, dtype=dtype)
    a = st.add_sequence(40)
    b = st.add_sequence(20)
    st.prefill_random()
    st.cache.erase(b)
    st.mirror.erase(b)
    before = bits(st.cache.kv_cache).copy()
    # rows: a live sequence, graph padding (slot 0), an erased slot (table row all -1)
    bidx = torch.tensor([a, 0, b, 0], dtype=torch.int64)
    pos = torch.tensor([[39], [0], [7], [5]], dtype=torch.int32)
    k = randn(st.gen, (4, 4, 1, 128), dtype)
    v = randn(st.gen, (4, 4, 1, 128), dtype)
    st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pos.to(DEV), batch_idx=bidx.to(DEV))
    got = bits(st.cache.kv_cache)
    P = st.P
    slot = int(st.mirror.page_table[a, 39 // P]) * P + 39 % P
    assert np.array_equal(got[0, 0, 0, :, slot], bits(k)[0, :, 0])
    assert np.array_equal(got[0, 1, 0, :, slot], bits(v)[0, :, 0])
    keep = np.ones(got.shape[4], dtype=bool)
    keep[:P] = False  # page 0 absorbs the redirected rows, its contents are unspecified
    keep[slot] = False
    assert np.array_equal(got[..., keep, :], before[..., keep, :])
    assert np.array_equal(got[0, 0, 0, :, 7], bits(k)[2, :, 0])  # erased slot: -1 clamped to page 0, offset 7


@pytest.mark.parametrize("dtype,D", [(torch.float32, 6), (torch.bfloat16, 10), (torch.float16, 36)])
def test_append_narrow_vector_paths(dtype, D):
    """Row sizes that are not multiples of 16 bytes take the 8/4/2-byte copy paths."""
    st = PagedState(4, n_pages=16, page_size=8, max_batch=4, Hc=2, D=D, dtype=dtype)
    st.add_sequence(19)
    st.add_sequence(30)
    k, v, bt, pt, _, _ = st.prefill_random()
    ref = oracle_pool(st)
    O.append_prefill(ref, 0, bits(k), bits(v), st.mirror.page_table, bt.numpy(), pt.numpy(), st.P)
    assert np.array_equal(bits(st.cache.kv_cache), ref)
    lens = torch.tensor(st.lens, dtype=torch.int32, device=DEV)
    g = ops.kv_gather(st.pool_planes()[0], st.cache.page_table, torch.tensor(st.slots, device=DEV), lens, st.P, 32)
    exp = O.gather_pages(ref[0, 0, 0], st.mirror.page_table, st.slots, st.lens, st.P, 32)
    assert np.array_equal(bits(g), exp)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gather_bit_exact_and_inverse_of_append(dtype):
    st = PagedState(5, n_pages=48, page_size=32, max_batch=8, Hc=4, D=128, dtype=dtype)
    for L in (1, 32, 33, 250, 64, 5):
        st.add_sequence(L)
    k, v, bt, pt, _, _ = st.prefill_random()
    pk, pv = st.pool_planes()
    slots = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    for lens_dtype in (torch.int32, torch.int64):
        lens = torch.tensor(st.lens, dtype=lens_dtype, device=DEV)
        max_len = 256
        gk = ops.kv_gather(pk, st.cache.page_table, slots, lens, st.P, max_len)
        gv = ops.kv_gather(pv, st.cache.page_table, slots, lens, st.P, max_len)
        pool_bits = bits(st.cache.kv_cache)
        ek = O.gather_pages(pool_bits[0, 0, 0], st.mirror.page_table, st.slots, st.lens, st.P, max_len)
        ev = O.gather_pages(pool_bits[0, 1, 0], st.mirror.page_table, st.slots, st.lens, st.P, max_len)
        assert np.array_equal(bits(gk), ek) and np.array_equal(bits(gv), ev)
    # round trip: what was appended comes back, in logical order
    off = 0
    kb = bits(k)
    for i, L in enumerate(st.lens):
        assert np.array_equal(bits(gk)[i, :, :L], kb[0, :, off:off + L])
        assert not bits(gk)[i, :, L:].any()
        off += L


def test_gather_into_a_strided_output():
    st = PagedState(6, n_pages=16, page_size=16, max_batch=4, Hc=2, D=64, dtype=torch.bfloat16)
    st.add_sequence(40)
    st.prefill_random()
    big = torch.full((1, 2, 64, 128), 7.0, dtype=torch.bfloat16, device=DEV)
    out = big[:, :, :48, :64]
    ops.kv_gather(st.pool_planes()[0], st.cache.page_table, torch.tensor(st.slots, device=DEV),
                  torch.tensor([40], device=DEV), st.P, 48, out=out)
    exp = O.gather_pages(bits(st.cache.kv_cache)[0, 0, 0], st.mirror.page_table, st.slots, [40], st.P, 48)
    assert np.array_equal(bits(out), exp)
    assert (big[:, :, 48:] == 7).all() and (big[..., 64:] == 7).all()  # outside the view untouched


def test_convert_block_ids_bit_exact():
    st = PagedState(7, n_pages=64, page_size=16, max_batch=10, Hc=1, D=64, dtype=torch.bfloat16)
    for L in (100, 400, 16, 330):
        st.add_sequence(L)
    gen = st.gen
    B, Hm, R, C = 4, 1, 2, 40
    idx = torch.randint(0, 64, (B, Hm, R, C), generator=gen, dtype=torch.int32)
    bidx = torch.tensor(st.slots, dtype=torch.int64)
    got = ops.convert_block_ids(idx.to(DEV), st.cache.page_table, bidx.to(DEV))
    exp = O.convert_block_ids(st.mirror.page_table, st.slots, idx.numpy(), 64)
    assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), exp)


def test_engine_decode_mask_conversion_matches_reference_semantics():
    """create_causal_blockmask -> per-step slice (as paged_inference.py:803-826 does) ->
    convert_logical_block_mask: physical block lists equal the oracle's."""
    from torch.nn.attention.flex_attention import BlockMask

    P, Lmax = 16, 256
    st = PagedState(8, n_pages=64, page_size=P, max_batch=6, Hc=1, D=64, dtype=torch.bfloat16)
    for L in (100, 17, 256, 33):
        st.add_sequence(L)
    cache = st.cache
    full = cache.create_causal_blockmask(B=6, L=Lmax)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos = torch.tensor([L - 1 for L in st.lens], dtype=torch.int32, device=DEV)
    blk = pos // P
    B = 4
    step = BlockMask.from_kv_blocks(
        full.kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.kv_indices[bidx, :, blk].view(B, 1, 1, -1),
        full.full_kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.full_kv_indices[bidx, :, blk].view(B, 1, 1, -1),
        BLOCK_SIZE=full.BLOCK_SIZE, mask_mod=lambda b, h, q, kv: q + pos[b] >= kv, seq_lengths=(1, Lmax))
    conv = cache.convert_logical_block_mask(step, bidx)
    kvn, kvi, fn, fi = O.causal_block_structure(Lmax // P)
    rows = (pos // P).cpu().numpy()
    exp_p = O.convert_block_ids(st.mirror.page_table, st.slots, kvi[rows][:, None, None, :], 64)
    exp_f = O.convert_block_ids(st.mirror.page_table, st.slots, fi[rows][:, None, None, :], 64)
    assert np.array_equal(conv.kv_indices.cpu().numpy(), exp_p)
    assert np.array_equal(conv.full_kv_indices.cpu().numpy(), exp_f)
    assert conv.kv_num_blocks.flatten().tolist() == [1] * B
    assert conv.full_kv_num_blocks.flatten().tolist() == rows.tolist()
    assert conv.seq_lengths == (1, 64 * P)
    # every page the kernel will read is listed: full blocks then the partial one
    for b in range(B):
        n_full = int(rows[b])
        pages = conv.full_kv_indices[b, 0, 0, :n_full].tolist() + conv.kv_indices[b, 0, 0, :1].tolist()
        assert pages == st.mirror.page_table_cpu[st.slots[b]][: n_full + 1]


def test_large_append_round_trip_and_checksum():
    """Prefill-sized append (32768 tokens x 16 heads x 128 bf16 = 128 MiB per tensor):
    gather(append(x)) == x and an order-independent checksum of the pool equals that of the input."""
    dtype = torch.bfloat16
    T, H, D, P = 32768, 16, 128, 128
    st = PagedState(9, n_pages=T // P + 9, page_size=P, max_batch=10, Hc=H, D=D, dtype=dtype)
    lens = [4096, 8192, 1000, 12288, 7192]
    assert sum(lens) == T
    for L in lens:
        st.add_sequence(L)
    g = torch.Generator(device=DEV).manual_seed(9)
    k = torch.randn((1, H, T, D), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    v = torch.randn((1, H, T, D), generator=g, device=DEV, dtype=torch.float32).to(dtype)
    bidx = torch.cat([torch.full((L,), b, dtype=torch.int64) for b, L in zip(st.slots, lens)])[None].to(DEV)
    pos = torch.cat([torch.arange(L, dtype=torch.int64) for L in lens])[None].to(DEV)
    st.cache.insert_kv(0, k, v, input_pos=pos, batch_idx=bidx)
    pk, pv = st.pool_planes()
    slots = torch.tensor(st.slots, device=DEV)
    lens_t = torch.tensor(lens, device=DEV)
    gk = ops.kv_gather(pk, st.cache.page_table, slots, lens_t, P, max(lens))
    gv = ops.kv_gather(pv, st.cache.page_table, slots, lens_t, P, max(lens))
    off = 0
    for i, L in enumerate(lens):
        assert torch.equal(gk[i, :, :L].view(torch.int16), k[0, :, off:off + L].view(torch.int16))
        assert torch.equal(gv[i, :, :L].view(torch.int16), v[0, :, off:off + L].view(torch.int16))
        assert not gk[i, :, L:].any()
        off += L
    # nothing else was written: the pool holds exactly the appended rows (sum of bit patterns)
    assert int(pk.view(torch.int16).to(torch.int64).sum()) == int(k.view(torch.int16).to(torch.int64).sum())
    assert int(pv.view(torch.int16).to(torch.int64).sum()) == int(v.view(torch.int16).to(torch.int64).sum())


@pytest.mark.bigmem
def test_append_and_gather_with_more_than_2_32_vectors_in_a_launch():
    """Rows of 3 bf16 values move as 2-byte vectors, one per lane; 1 435 000 000 such rows are more than
    2^32 lanes in one launch, the case in which the kernels index their lanes with 64 bits.  One sequence
    whose pages lie in reverse order; checked on the GPU (the pool, read back page by page, is the
    input, and the gather returns it), bit for bit."""
    free, _ = torch.cuda.mem_get_info()
    assert free > 90e9, f"only {free / 1e9:.0f} GB of HBM free: this case holds about 60 GB"
    S, D, P = 1_435_000_000, 3, 128
    assert S * D > 2**32
    n_pages = -(-S // P)
    n_slots = n_pages * P
    g = torch.Generator(device=DEV).manual_seed(11)
    k = torch.randint(-32768, 32767, (1, 1, S, D), generator=g, device=DEV, dtype=torch.int16).view(torch.bfloat16)
    v = torch.randint(-32768, 32767, (1, 1, S, D), generator=g, device=DEV, dtype=torch.int16).view(torch.bfloat16)
    pool_k = torch.zeros((1, n_slots, D), dtype=torch.bfloat16, device=DEV)
    pool_v = torch.zeros((1, n_slots, D), dtype=torch.bfloat16, device=DEV)
    page_table = torch.zeros((2, n_pages), dtype=torch.int64, device=DEV)
    page_table[1] = torch.arange(n_pages - 1, -1, -1, device=DEV)
    bidx = torch.ones(1, dtype=torch.int64, device=DEV)
    pos = torch.arange(S, dtype=torch.int32, device=DEV)[None]
    ops.kv_append(pool_k, pool_v, k, v, page_table, bidx, pos, P, clamp_negative=False)
    del pos
    for pool, src in ((pool_k, k), (pool_v, v)):
        back = pool.view(n_pages, P, D).flip(0).reshape(n_slots, D)[:S]
        assert torch.equal(back.view(torch.int16), src[0, 0].view(torch.int16))
        del back
    lens = torch.tensor([S], dtype=torch.int64, device=DEV)
    got = ops.kv_gather(pool_k, page_table, bidx, lens, P, S)
    assert torch.equal(got[0, 0].view(torch.int16), k[0, 0].view(torch.int16))
