"""GPU parity: decode on a cache that stores one head per query head with identical V copies inside a
group (the reference's repeat_kv layout, model.py:112-114; K copies differ through the per-head rotary
angles).  kv_rep > 1 reads V once per group; the result must equal the plain read of the same cache."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, bits, f64, randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float32: (2e-5, 2e-5)}


def expanded_state(seed, rep, dtype, P, lens, Hkv=2, D=128):
    Hq = Hkv * rep
    st = PagedState(seed, n_pages=sum(-(-(L + 1) // P) for L in lens) + 3, page_size=P, max_batch=len(lens) + 2,
                    Hc=Hq, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    total = sum(lens)
    k = randn(st.gen, (1, Hq, total, D), dtype)                                   # every head its own K
    v = randn(st.gen, (1, Hkv, total, D), dtype).repeat_interleave(rep, dim=1)    # V copied inside a group
    bidx = torch.cat([torch.full((L,), b) for b, L in zip(st.slots, lens)])[None]
    pos = torch.cat([torch.arange(L) for L in lens])[None]
    if total:
        st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pos.to(DEV), batch_idx=bidx.to(DEV))
    return st, Hq


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("rep,P", [(2, 128), (4, 64), (2, 24)])
def test_shared_v_read_equals_the_plain_read(dtype, rep, P):
    lens = [0, 1, 63, 64, 700, 1500, 333]
    st, Hq = expanded_state(51, rep, dtype, P, lens)
    B = len(lens)
    q = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV) - 1
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pk, pv = st.pool_planes()
    args = (q, pk, pv, st.cache.page_table, bidx, pos, P, 1536)
    for split in (256, 2048):
        plain = ops.paged_decode(*args, split_tokens=split)
        shared = ops.paged_decode(*args, split_tokens=split, kv_rep=rep)
        atol, rtol = TOL[dtype]
        np.testing.assert_allclose(f64(shared[0]), f64(plain[0]), atol=atol, rtol=rtol)
        np.testing.assert_allclose(f64(shared[1]), f64(plain[1]), atol=1e-4, rtol=1e-5)
        if rep == 2:  # same loads in flight, same folding order per head: the same bits
            assert np.array_equal(bits(shared[0]), bits(plain[0])) and torch.equal(shared[1], plain[1])
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, pos.cpu().numpy(), P)
    np.testing.assert_allclose(f64(shared[0]), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(shared[1]), el, atol=max(atol * 0.1, 2e-5), rtol=rtol)


@pytest.mark.parametrize("rep", [2, 4])
def test_shared_v_with_fused_append(rep):
    dtype, P = torch.bfloat16, 32
    lens = [0, 31, 32, 500]
    results = []
    for mode in ("separate", "fused-shared"):
        st, Hq = expanded_state(52, rep, dtype, P, lens)
        B = len(lens)
        k1 = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
        v1 = randn(st.gen, (B, Hq // rep, 1, 128), dtype).repeat_interleave(rep, dim=1).to(DEV)
        q = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
        pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
        bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
        pk, pv = st.pool_planes()
        if mode == "separate":
            st.cache.insert_kv(0, k1, v1, input_pos=pos.view(B, 1), batch_idx=bidx)
            out, lse = ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, P, 512, split_tokens=128)
        else:
            out, lse = ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, P, 512, split_tokens=128,
                                        k_new=k1, v_new=v1, kv_rep=rep)
        results.append((st.cache.kv_cache.clone(), out, lse))
    assert np.array_equal(bits(results[0][0]), bits(results[1][0]))  # every K head and every V copy written
    np.testing.assert_allclose(f64(results[1][1]), f64(results[0][1]), atol=2e-2, rtol=1e-2)
    np.testing.assert_allclose(f64(results[1][2]), f64(results[0][2]), atol=1e-4, rtol=1e-5)


def test_kv_rep_is_validated():
    st, Hq = expanded_state(53, 2, torch.bfloat16, 16, [20])
    q = randn(st.gen, (1, Hq, 1, 128), torch.bfloat16).to(DEV)
    pk, pv = st.pool_planes()
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos = torch.tensor([19], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="kv_rep"):
        ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, 16, 64, kv_rep=3)
    with pytest.raises(RuntimeError, match="one head per query head"):
        ops.paged_decode(q, pk[:2], pv[:2], st.cache.page_table, bidx, pos, 16, 64, kv_rep=2)


def test_shared_v_and_sink_gate_through_the_even_cut():
    """A launch of more workgroups than the GPU holds at once (80 sequences x 8 groups x 8 splits) is cut
    into equal chunks of the flattened contexts; the shared-V read and the sink gate go through that path
    and its merge pass too."""
    dtype, P, rep, B = torch.bfloat16, 64, 2, 80
    gen = torch.Generator().manual_seed(53)
    lens = torch.randint(1, 500, (B,), generator=gen).tolist()
    lens[0], lens[1] = 0, 511
    st, Hq = expanded_state(53, rep, dtype, P, lens, Hkv=8)
    q = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV) - 1
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    sinks = torch.linspace(-2.0, 2.0, Hq, device=DEV)
    pk, pv = st.pool_planes()
    args = (q, pk, pv, st.cache.page_table, bidx, pos, P, 512)
    out, lse = ops.paged_decode(*args, split_tokens=64, kv_rep=rep)
    gated, lse_g = ops.paged_decode(*args, split_tokens=64, kv_rep=rep, sinks=sinks)
    atol, rtol = TOL[dtype]
    eo, el = O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, pos.cpu().numpy(), P)
    np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse), el, atol=max(atol * 0.1, 2e-5), rtol=rtol)
    assert torch.equal(lse_g, lse)
    gate = 1.0 / (1.0 + np.exp(f64(sinks)[None, :, None] - f64(lse)))
    np.testing.assert_allclose(f64(gated), f64(out) * gate[..., None], atol=atol, rtol=rtol)
    assert not f64(out)[0].any() and np.isneginf(f64(lse)[0]).all()  # the sequence without keys


@pytest.mark.parametrize("fused", [False, True], ids=["append-launch", "append-in-attention"])
def test_a_cache_that_knows_its_v_copies_decodes_through_the_reference_call(fused):
    """`install(kv_rep=2)` gives every new cache kv_rep = 2; the unchanged call sequence of the reference
    (insert_kv with expanded K/V, compiled_flex_attn_decode on the returned pool views) then reads V once per
    group and returns what the plain read returns -- also when the append is left to the attention launch, which
    then writes every copy of the new V row."""
    from torch.nn.attention.flex_attention import AuxRequest

    from falcon_perception_amd import attention as A

    dtype, P, rep = torch.bfloat16, 32, 2
    lens = [5, 64, 300, 31]
    st, Hq = expanded_state(57, rep, dtype, P, lens)
    cache = st.cache
    cache.fuse_decode_append = fused
    B = len(lens)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
    k = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
    v = randn(st.gen, (B, Hq // rep, 1, 128), dtype).repeat_interleave(rep, dim=1).to(DEV)
    q = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
    logical = cache.create_causal_blockmask(B=B, L=512)
    mask = cache.convert_logical_block_mask(logical, bidx)  # the kernel takes positions from the step, not the mask
    results = {}
    for r in (1, rep):
        cache.kv_rep = r
        K, V = cache.insert_kv(0, k, v, input_pos=pos.view(B, 1), batch_idx=bidx)
        assert (cache.last_decode_step.k_new is not None) == fused
        out, aux = A.compiled_flex_attn_decode(q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
        assert cache.last_decode_step.k_new is None
        results[r] = (out.clone(), aux.lse.clone())
    assert cache.v_copies_are_identical()
    assert torch.equal(results[1][0], results[rep][0]) and torch.equal(results[1][1], results[rep][1])
    eo, el = O.decode_attention(f64(q), f64(K[0]), f64(V[0]), st.mirror.page_table, st.slots, np.array(lens), P)
    np.testing.assert_allclose(f64(results[rep][0]), eo, atol=2e-2, rtol=1e-2)
