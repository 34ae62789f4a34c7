"""GPU parity: split-K paged decode attention against the float64 oracle.

Tolerance (north star): 2e-2 absolute / 1e-2 relative for bf16; fp32 and fp16 are
held to tighter bounds written next to each check.
"""

import math

import numpy as np
import pytest
import torch
from torch.nn.attention.flex_attention import AuxRequest, BlockMask

from falcon_perception_amd import attention as A
from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, f64, randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float16: (2e-3, 2e-3), torch.float32: (2e-5, 2e-5)}


def run_decode(st, q, pos, **kw):
    pk, pv = st.pool_planes()
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    max_ctx = kw.pop("max_context", st.cache.n_pages * st.P)
    return ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), st.P, max_ctx, **kw)


def oracle_decode(st, q, pos):
    pk, pv = st.pool_planes()
    return O.decode_attention(f64(q), f64(pk), f64(pv), st.mirror.page_table, st.slots, pos.numpy(), st.P)


def assert_close(out, lse, eo, el, dtype):
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse), el, atol=max(atol * 0.1, 1e-5), rtol=rtol)


def test_cfg1_cpu_reference_shape_fp32():
    """BASELINE configs[0]: 64 pages x 64, 8 heads x 64, fp32, batch 4, contexts U[64,512],
    append one token per sequence then decode."""
    st = PagedState(1, n_pages=64, page_size=64, max_batch=8, Hc=8, D=64, dtype=torch.float32)
    lens = torch.randint(64, 513, (4,), generator=st.gen).tolist()
    for L in lens:
        st.add_sequence(L + 1)  # room for the appended token
    st.lens = lens
    st.prefill_random()
    k = randn(st.gen, (4, 8, 1, 64), torch.float32)
    v = randn(st.gen, (4, 8, 1, 64), torch.float32)
    q = randn(st.gen, (4, 8, 1, 64), torch.float32)
    pos = torch.tensor(lens, dtype=torch.int32)  # the new token's position
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pos.view(4, 1).to(DEV), batch_idx=bidx)
    out, lse = run_decode(st, q, pos)
    eo, el = oracle_decode(st, q, pos)
    assert_close(out, lse, eo, el, torch.float32)
    assert out.dtype == torch.float32 and lse.dtype == torch.float32 and lse.shape == (4, 8, 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G", [1, 2, 4, 8])
@pytest.mark.parametrize("P", [16, 128, 24])
def test_context_boundaries_and_gqa(dtype, D, G, P):
    """Contexts at every page and split boundary, for every template instance of the split-by-split pass:
    one split that stores its result directly (split_tokens 512), several splits and the merge pass; page
    sizes whose rows a load instruction covers exactly (128), smaller (16) and no power of two (24)."""
    lens = [1, 2, P - 1, P, P + 1, 4 * P, 4 * P + 1, 63, 64, 65, 300]
    st = PagedState(2, n_pages=sum(-(-L // P) for L in lens) + 4, page_size=P, max_batch=12, Hc=2, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (len(lens), 2 * G, 1, D), dtype)
    pos = torch.tensor([L - 1 for L in lens], dtype=torch.int32)
    eo, el = oracle_decode(st, q, pos)
    for split in (0, 64, 128, 512):
        out, lse = run_decode(st, q, pos, split_tokens=split, max_context=max(lens) + 20)
        assert_close(out, lse, eo, el, dtype)


def test_no_visible_key_and_int64_positions():
    dtype = torch.bfloat16
    st = PagedState(3, n_pages=32, page_size=16, max_batch=6, Hc=2, D=128, dtype=dtype)
    for L in (40, 70, 9):
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (3, 4, 1, 128), dtype)
    pos = torch.tensor([39, -1, 8], dtype=torch.int64)
    for ctx in (64, 512):  # single-split (direct) and split-K + merge paths
        out, lse = run_decode(st, q, pos, max_context=ctx)
        eo, el = oracle_decode(st, q, pos)
        assert_close(out[[0, 2]], lse[[0, 2]], eo[[0, 2]], el[[0, 2]], dtype)
        assert not out[1].any() and torch.isneginf(lse[1]).all()


def test_page_permutation_and_split_invariance():
    """Same logical content under two page tables gives identical results bit for bit;
    different split sizes agree to fp32 rounding."""
    dtype = torch.bfloat16
    outs = []
    for shuffle in (False, True):
        st = PagedState(4, n_pages=64, page_size=32, max_batch=6, Hc=4, D=128, dtype=dtype, shuffle=shuffle)
        gen = torch.Generator().manual_seed(44)
        st.gen = gen  # identical K/V/q for both layouts
        for L in (500, 37, 960):
            st.add_sequence(L)
        st.prefill_random()
        q = randn(gen, (3, 8, 1, 128), dtype)
        pos = torch.tensor([499, 36, 959], dtype=torch.int32)
        outs.append(run_decode(st, q, pos, split_tokens=256, max_context=1024))
        if shuffle:
            o64 = run_decode(st, q, pos, split_tokens=64, max_context=1024)
            o1k = run_decode(st, q, pos, split_tokens=1024, max_context=1024)
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    np.testing.assert_allclose(f64(o64[1]), f64(o1k[1]), atol=1e-5, rtol=1e-5)
    np.testing.assert_allclose(f64(o64[0]), f64(o1k[0]), atol=8e-3, rtol=8e-3)  # one bf16 ulp of the output


def test_strided_query_and_preallocated_outputs():
    dtype = torch.bfloat16
    st = PagedState(5, n_pages=32, page_size=16, max_batch=4, Hc=2, D=128, dtype=dtype)
    st.add_sequence(130)
    st.add_sequence(77)
    st.prefill_random()
    # q as the model produces it: [B, S, H, D] memory viewed as [B, H, S, D]
    q = randn(st.gen, (2, 1, 4, 128), dtype).to(DEV).permute(0, 2, 1, 3)
    assert not q.is_contiguous() or q.shape[2] == 1
    pos = torch.tensor([129, 76], dtype=torch.int32)
    out = torch.zeros((2, 1, 4, 128), dtype=dtype, device=DEV).permute(0, 2, 1, 3)
    lse = torch.zeros((2, 4, 1), dtype=torch.float32, device=DEV)
    r_out, r_lse = run_decode(st, q, pos, out=out, lse=lse, max_context=256)
    assert r_out.data_ptr() == out.data_ptr()
    eo, el = oracle_decode(st, q.cpu(), pos)
    assert_close(out, lse, eo, el, dtype)


def test_cfg2_serving_shape_bf16():
    """BASELINE configs[1] at full size: batch 64, 16 q / 8 kv heads, D 128, page 128,
    contexts 1024 + U[64,3072], fragmented 4096-page pool."""
    import bench

    case = bench.make_decode_case("cfg2", device=DEV)
    out, lse = case.run()
    f32 = lambda t: t.float().cpu().numpy()  # exact for bf16; the oracle widens per sequence
    eo, el = O.decode_attention(f64(case.q), f32(case.pool_k), f32(case.pool_v), case.page_table.cpu().numpy(),
                                case.batch_idx.cpu().numpy(), case.input_pos.cpu().numpy(), case.page_size)
    assert_close(out, lse, eo, el, torch.bfloat16)


def test_attention_callable_with_engine_masks():
    """The reference's call: insert_kv then compiled_flex_attn_decode(q, K, V, block_mask, return_aux)
    (model.py:150-162) with the mask built as paged_inference.py:783-848 builds it."""
    dtype = torch.bfloat16
    P, Lmax, H, D = 16, 256, 4, 128
    st = PagedState(6, n_pages=64, page_size=P, max_batch=8, Hc=H, D=D, dtype=dtype)
    lens = [100, 17, 255, 33]
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    cache = st.cache
    full = cache.create_causal_blockmask(B=8, L=Lmax)
    # two padded rows with batch slot 0 as CUDA-graph buckets have (paged_inference.py:970-992)
    bidx = torch.tensor(st.slots + [0, 0], dtype=torch.int64, device=DEV)
    input_pos_all = torch.zeros(8, dtype=torch.int32, device=DEV)
    input_pos_all[torch.tensor(st.slots, device=DEV)] = torch.tensor(lens, dtype=torch.int32, device=DEV)
    pos = input_pos_all[bidx]
    B = 6
    blk = pos // P
    step = BlockMask.from_kv_blocks(
        full.kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.kv_indices[bidx, :, blk].view(B, 1, 1, -1),
        full.full_kv_num_blocks[bidx, :, blk].view(B, 1, 1), full.full_kv_indices[bidx, :, blk].view(B, 1, 1, -1),
        BLOCK_SIZE=full.BLOCK_SIZE, mask_mod=lambda b, h, q, kv: q + pos[b] >= kv, seq_lengths=(1, Lmax))
    mask = cache.convert_logical_block_mask(step, bidx)
    k = randn(st.gen, (B, H, 1, D), dtype).to(DEV)
    v = randn(st.gen, (B, H, 1, D), dtype).to(DEV)
    q = randn(st.gen, (B, H, 1, D), dtype).to(DEV)
    K, V = cache.insert_kv(0, k, v, input_pos=pos.view(B, 1), batch_idx=bidx)
    out, aux = A.compiled_flex_attn_decode(q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True),
                                           kernel_options={"BLOCK_M": 64, "BLOCK_N": 64, "num_stages": 1})
    assert out.shape == (B, H, 1, D) and aux.lse.shape == (B, H, 1)
    eo, el = O.decode_attention(f64(q[:4]), f64(K[0]), f64(V[0]), cache.page_table.cpu().numpy(),
                                st.slots, np.array(lens), P)
    assert_close(out[:4], aux.lse[:4], eo, el, dtype)
    assert torch.isfinite(out.float()).all()  # padded rows read page 0 and stay finite
    # the same step through a captured HIP graph, replayed with new positions
    g = torch.cuda.CUDAGraph()
    static_q = q.clone()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        A.compiled_flex_attn_decode(static_q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    torch.cuda.current_stream().wait_stream(s)
    with torch.cuda.graph(g):
        g_out, g_aux = A.compiled_flex_attn_decode(static_q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
    for trial in range(3):
        static_q.copy_(randn(st.gen, (B, H, 1, D), dtype))
        g.replay()
        torch.cuda.synchronize()
        e_out, e_aux = A.compiled_flex_attn_decode(static_q, K, V, block_mask=mask, return_aux=AuxRequest(lse=True))
        assert torch.equal(g_out, e_out) and torch.equal(g_aux.lse, e_aux.lse)


def test_partial_then_merge_equals_the_fused_call():
    dtype = torch.bfloat16
    st = PagedState(7, n_pages=96, page_size=32, max_batch=6, Hc=2, D=128, dtype=dtype)
    for L in (700, 64, 1300):
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (3, 4, 1, 128), dtype)
    pos = torch.tensor([699, 63, 1299], dtype=torch.int32)
    ws = torch.zeros(ops.decode_workspace_bytes(3, 4, 128, 1408, 256), dtype=torch.uint8, device=DEV)
    both = run_decode(st, q, pos, split_tokens=256, max_context=1408, workspace=ws)
    out = torch.zeros_like(both[0])
    lse = torch.zeros_like(both[1])
    run_decode(st, q, pos, split_tokens=256, max_context=1408, workspace=ws, out=out, lse=lse, phase="partial")
    assert not out.any()  # the partial pass leaves out untouched when there are several splits
    run_decode(st, q, pos, split_tokens=256, max_context=1408, workspace=ws, out=out, lse=lse, phase="merge")
    assert torch.equal(out, both[0]) and torch.equal(lse, both[1])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("ctx", [320, 1280])
def test_fused_append_decode_equals_append_then_decode(dtype, ctx):
    """fp_paged_decode_append: same pool bits as the append kernel, same attention as the oracle.
    Contexts include L = 1 (only the new token), split and page boundaries."""
    P = 16
    G = 2
    outs = []
    lens = [0, 1, P - 1, P, P + 1, 63, 64, 65, 127, 128, 300]  # tokens cached before the step
    for fused in (False, True):
        st = PagedState(8, n_pages=80, page_size=P, max_batch=13, Hc=2, D=128, dtype=dtype)
        for L in lens:
            st.add_sequence(L + 1)
        st.lens = lens
        st.prefill_random()
        B = len(lens)
        k1 = randn(st.gen, (B, 2, 1, 128), dtype)
        v1 = randn(st.gen, (B, 2, 1, 128), dtype)
        q = randn(st.gen, (B, 2 * G, 1, 128), dtype)
        pos = torch.tensor(lens, dtype=torch.int32)
        bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
        pk, pv = st.pool_planes()
        if fused:
            out, lse = ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), P, ctx,
                                        split_tokens=64, k_new=k1.to(DEV), v_new=v1.to(DEV))
        else:
            st.cache.insert_kv(0, k1.to(DEV), v1.to(DEV), input_pos=pos.view(B, 1).to(DEV), batch_idx=bidx)
            out, lse = ops.paged_decode(q.to(DEV), pk, pv, st.cache.page_table, bidx, pos.to(DEV), P, ctx,
                                        split_tokens=64)
        outs.append((out, lse, st.cache.kv_cache.clone()))
        if fused:
            eo, el = oracle_decode(st, q, pos)
            assert_close(out, lse, eo, el, dtype)
    assert torch.equal(outs[0][2].view(torch.uint8), outs[1][2].view(torch.uint8))  # pools bit-identical
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(outs[1][0]), f64(outs[0][0]), atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(outs[1][1]), f64(outs[0][1]), atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype,D", [(torch.bfloat16, 128), (torch.float32, 64)], ids=str)
@pytest.mark.parametrize("longest,split_tokens,n_splits", [(1300, 192, 7), (1300, 128, 11), (1300, 64, 21), (6000, 64, 94)])
def test_merge_pass_with_few_and_with_many_splits(longest, split_tokens, n_splits, dtype, D):
    """The merge pass has three forms: every partial requested at once (up to 8 splits), one wavefront
    walking batches of 8 (up to 16), and eight wavefronts sharing the batches (beyond; with 94 splits
    some of them take two batches and some one).  Each with sequences that fill all, some or one of the
    splits, and one without any key."""
    st = PagedState(21, n_pages=256, page_size=32, max_batch=8, Hc=2, D=D, dtype=dtype)
    for L in (longest, 65, 500, 1):
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (4, 4, 1, D), dtype)
    pos = torch.tensor([longest - 1, 64, 499, -1], dtype=torch.int32)
    assert -(-longest // split_tokens) == n_splits
    out, lse = run_decode(st, q, pos, split_tokens=split_tokens, max_context=longest)
    eo, el = oracle_decode(st, q[:3], pos[:3])
    assert_close(out[:3], lse[:3], eo, el, dtype)
    assert not out[3].any() and torch.isneginf(lse[3]).all()


@pytest.mark.parametrize("dtype,D,P,G", [(torch.bfloat16, 128, 64, 2), (torch.float32, 64, 16, 1), (torch.float16, 128, 48, 4)],
                         ids=str)
def test_a_launch_larger_than_the_gpu_is_cut_evenly(dtype, D, P, G):
    """8 cache heads x 72 sequences x 8 splits = 4608 workgroups, more than the GPU holds at once: the
    contexts are laid end to end and cut into equal chunks instead (about 190 tokens here), so chunks span
    several short sequences and long sequences span several chunks.  Sequences of 1 token, of exactly one
    chunk-rounding unit, one without any key and one at the maximum; fused append; the two passes called
    separately; the same launch replayed from a graph."""
    B, Hc, split, ctx = 72, 8, 64, 512
    st = PagedState(33, n_pages=B * (-(-ctx // P)) + 8, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    lens = torch.randint(0, ctx - 1, (B,), generator=st.gen).tolist()  # tokens cached before the step
    lens[0], lens[1], lens[2], lens[3], lens[40] = ctx - 1, 0, 63, 64, 0
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    k_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    v_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32)  # the new token's position
    kw = dict(split_tokens=split, max_context=ctx)
    out, lse = run_decode(st, q, pos, k_new=k_new, v_new=v_new, **kw)
    eo, el = oracle_decode(st, q, pos)  # the pool now holds the new rows
    assert_close(out, lse, eo, el, dtype)
    # without the append (the rows are in the pool), one sequence masked out, passes called separately
    pos2 = pos.clone()
    pos2[5] = -1
    need = ops.decode_workspace_bytes(B, Hc * G, D, ctx, split)
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device=DEV)
    run_decode(st, q, pos2, workspace=ws, phase="partial", **kw)
    out2, lse2 = run_decode(st, q, pos2, workspace=ws, phase="merge", **kw)
    keep = [i for i in range(B) if i != 5]  # their chunks lie elsewhere now: same values within rounding
    assert_close(out2[keep], lse2[keep], eo[keep], el[keep], dtype)
    assert not out2[5].any() and torch.isneginf(lse2[5]).all()
    # from a graph, replayed
    qd, bidx, posd = q.to(DEV), torch.tensor(st.slots, dtype=torch.int64, device=DEV), pos.to(DEV)
    pk, pv = st.pool_planes()
    out_g, lse_g = torch.empty_like(out), torch.empty_like(lse)
    call = lambda: ops.paged_decode(qd, pk, pv, st.cache.page_table, bidx, posd, st.P, ctx, split_tokens=split,
                                    workspace=ws, out=out_g, lse=lse_g, k_new=k_new, v_new=v_new)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()
    torch.cuda.current_stream().wait_stream(side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call()
    for _ in range(3):
        out_g.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, out) and torch.equal(lse_g, lse)


@pytest.mark.parametrize("B,ctx", [(50, 128), (100, 128), (97, 192), (200, 256)])
def test_no_pass_writes_outside_the_workspace_it_asked_for(B, ctx):
    """Launches around the point where the even cut takes over (8 heads x B sequences x 2 to 4 splits
    against the workgroups the GPU holds at once): the even cut needs a workspace row per (chunk +
    sequence) and must leave the launch alone where the rows asked for split by split would not hold them.
    The workspace sits inside a larger buffer whose remainder must come back untouched."""
    dtype, D, P, Hc, G, split = torch.bfloat16, 128, 32, 8, 2, 64
    st = PagedState(35, n_pages=B * (-(-ctx // P)) + 8, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    lens = torch.randint(1, ctx, (B,), generator=st.gen).tolist()
    for L in lens:
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    pos = torch.tensor(lens, dtype=torch.int32) - 1
    need = ops.decode_workspace_bytes(B, Hc * G, D, ctx, split)
    guard = 1 << 20
    buf = torch.full((need + guard,), 0x5A, dtype=torch.uint8, device=DEV)
    out, lse = run_decode(st, q, pos, workspace=buf[:need], split_tokens=split, max_context=ctx)
    assert bool((buf[need:] == 0x5A).all())
    eo, el = oracle_decode(st, q, pos)
    assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("split,B", [(64, 3), (0, 3), (64, 80)])
def test_fused_append_beyond_max_context_leaves_the_pool_alone(split, B):
    """A sequence whose new position is max_context or more lies outside what the launch was sized for: its
    fresh row is neither stored (the slot of position max_context - 1 holds a valid row) nor attended; the
    other sequences of the step append as usual.  Also on the evenly cut launch (B = 80)."""
    dtype, P, Hc, G, D, ctx = torch.bfloat16, 16, 2, 2, 128, 256
    st = PagedState(41, n_pages=B * 18 + 4, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    lens = [ctx, ctx + 5, 100] + [37 + i for i in range(B - 3)]  # tokens cached before the step
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    before = st.cache.kv_cache.clone()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    k_new = randn(st.gen, (B, Hc, 1, D), dtype)
    v_new = randn(st.gen, (B, Hc, 1, D), dtype)
    pos = torch.tensor(lens, dtype=torch.int32)
    out, lse = run_decode(st, q, pos, k_new=k_new.to(DEV), v_new=v_new.to(DEV), split_tokens=split, max_context=ctx)
    # expected pool: the rows of sequences 2.. appended by the oracle's decode append, 0 and 1 untouched
    ref = before.double().cpu().numpy()
    O.append_decode(ref, 0, f64(k_new[2:]), f64(v_new[2:]), st.mirror.page_table, np.array(st.slots[2:]),
                    np.array(lens[2:])[:, None], P)
    assert np.array_equal(st.cache.kv_cache.double().cpu().numpy(), ref)
    # expected attention: positions 0 .. ctx - 1 for the two sequences beyond, the full context for the rest
    seen = pos.clone()
    seen[:2] = ctx - 1
    eo, el = oracle_decode(st, q, seen)
    assert_close(out, lse, eo, el, dtype)


def test_one_position_and_slot_per_sequence_is_required():
    st = PagedState(42, n_pages=8, page_size=16, max_batch=6, Hc=1, D=64, dtype=torch.bfloat16)
    for L in (5, 9, 20):
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (3, 1, 1, 64), torch.bfloat16)
    with pytest.raises(RuntimeError, match="one entry per sequence"):
        run_decode(st, q, torch.tensor([4, 8], dtype=torch.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("G", [1, 2, 4, 8])
@pytest.mark.parametrize("P", [64, 24], ids=["aligned-pages", "odd-pages"])
def test_every_instance_of_the_even_cut(dtype, D, G, P):
    """One launch per template instance of the split-K pass in its even-cut form (4 cache heads x 96 sequences
    x 8 splits = 3072 workgroups, more than the GPU holds at once), fused append included; where a workgroup
    serves several query heads, also on the expanded cache (one cached head per query head, V copies
    identical, read once per group)."""
    B, Hc, split, ctx = 96, 4, 64, 512
    lens = torch.randint(0, ctx - 1, (B,), generator=torch.Generator().manual_seed(70 + G)).tolist()
    lens[0], lens[1], lens[2] = ctx - 1, 0, 64
    for rep in (1, G) if G in (2, 4) else (1,):  # a group read as one is 2 or 4 heads wide
        H_pool = Hc * rep
        st = PagedState(60 + G, n_pages=B * (-(-ctx // P)) + 8, page_size=P, max_batch=B + 2, Hc=H_pool, D=D, dtype=dtype)
        for L in lens:
            st.add_sequence(L + 1)
        st.lens = lens
        st.prefill_random()
        if rep > 1:  # make the V copies of a group identical, as repeat_kv leaves them
            _, pv = st.pool_planes()
            pv.copy_(pv.view(Hc, rep, *pv.shape[1:])[:, :1].expand(Hc, rep, *pv.shape[1:]).reshape(pv.shape).clone())
        q = randn(st.gen, (B, Hc * G, 1, D), dtype)
        k_new = randn(st.gen, (B, H_pool, 1, D), dtype).to(DEV)
        v_new = randn(st.gen, (B, Hc, 1, D), dtype).repeat_interleave(rep, dim=1).to(DEV)
        pos = torch.tensor(lens, dtype=torch.int32)
        out, lse = run_decode(st, q, pos, k_new=k_new, v_new=v_new, split_tokens=split, max_context=ctx, kv_rep=rep)
        eo, el = oracle_decode(st, q, pos)  # the pool now holds the new rows
        assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("B", [1024, 1025, 3000])
def test_more_sequences_than_the_even_cut_keeps_in_lds(B):
    """The even cut holds the lengths of at most 1024 sequences; one more and the launch goes split by split
    (9000 and more workgroups).  Short contexts, some empty, fused append."""
    dtype, P, D, Hc, G = torch.bfloat16, 16, 64, 2, 2
    gen = torch.Generator().manual_seed(B)
    lens = torch.randint(0, 200, (B,), generator=gen).tolist()
    lens[3], lens[B - 1] = 0, 199
    st = PagedState(B, n_pages=sum(-(-(L + 1) // P) for L in lens) + 4, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    for L in lens:
        st.add_sequence(L + 1)
    st.lens = lens
    st.prefill_random()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype)
    k_new, v_new = randn(st.gen, (B, Hc, 1, D), dtype).to(DEV), randn(st.gen, (B, Hc, 1, D), dtype).to(DEV)
    pos = torch.tensor(lens, dtype=torch.int32)
    out, lse = run_decode(st, q, pos, k_new=k_new, v_new=v_new, split_tokens=64, max_context=256)
    eo, el = oracle_decode(st, q, pos)
    assert_close(out, lse, eo, el, dtype)


@pytest.mark.parametrize("P", [128, 16])
def test_one_sequence_of_a_million_tokens(P):
    """Context 1 000 000 on one cache head: thousands of splits (or long even-cut chunks with more page ids
    than a workgroup keeps), positions near 2^20; against the float64 oracle."""
    dtype, D, ctx = torch.bfloat16, 128, 1_000_000
    st = PagedState(5, n_pages=-(-(ctx + 1) // P) + 3, page_size=P, max_batch=3, Hc=1, D=D, dtype=dtype)
    st.add_sequence(ctx)
    pk, pv = st.pool_planes()
    g = torch.Generator(device=DEV).manual_seed(5)
    pk.copy_(torch.randn(pk.shape, generator=g, device=DEV, dtype=torch.float32))
    pv.copy_(torch.randn(pv.shape, generator=g, device=DEV, dtype=torch.float32))
    q = randn(st.gen, (1, 2, 1, D), dtype)
    pos = torch.tensor([ctx - 1], dtype=torch.int32)
    eo, el = oracle_decode(st, q, pos)
    for split in (0, 256, 65536 if P == 128 else 8192):
        out, lse = run_decode(st, q, pos, split_tokens=split, max_context=ctx)
        assert_close(out, lse, eo, el, dtype)
    if P == 16:  # a split holds the ids of at most 1022 pages: a wider one is refused, not truncated
        with pytest.raises(RuntimeError, match="spans more than"):
            run_decode(st, q, pos, split_tokens=65536, max_context=ctx)
