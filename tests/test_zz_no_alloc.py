"""GPU: the allocation-free decode entry point (fp_paged_decode_noalloc) against fp_paged_decode.

Two calls in a row share the library's scratch array, the second with a smaller input: what the first
call left there must not leak into the second.  Outputs must be bit-identical to fp_paged_decode with a
caller-owned workspace (same kernels, same partial results, another buffer)."""

import pytest
import torch

from falcon_perception_amd import _native, ops
from tests.gpu_cases import DEV, PagedState, randn

pytestmark = pytest.mark.gpu


def case(seed, B, ctx, Hc, G, D, P, dtype):
    st = PagedState(seed, n_pages=B * (-(-ctx // P)) + 4, page_size=P, max_batch=B + 2, Hc=Hc, D=D, dtype=dtype)
    lens = torch.randint(1, ctx + 1, (B,), generator=st.gen).tolist()
    lens[0] = ctx
    for L in lens:
        st.add_sequence(L)
    st.prefill_random()
    q = randn(st.gen, (B, Hc * G, 1, D), dtype).to(DEV)
    pos = torch.tensor([L - 1 for L in lens], dtype=torch.int32, device=DEV)
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    return st, q, pos, bidx


def both_ways(st, q, pos, bidx, ctx, split):
    pk, pv = st.pool_planes()
    ref_out, ref_lse = ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, ctx, split_tokens=split)
    out = torch.full_like(ref_out, float("nan"))
    lse = torch.full_like(ref_lse, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    ops.paged_decode_noalloc(q, pk, pv, st.cache.page_table, bidx, pos, st.P, ctx, out, lse, split_tokens=split)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before  # the wrapper took nothing from torch's allocator either
    assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse)


def test_two_calls_in_a_row_the_second_smaller():
    # 72 sequences x 8 heads x 8 splits: the evenly cut launch; then 3 sequences split by split, whose few
    # partial rows lie where the first call's lay
    big = case(51, 72, 512, 8, 2, 128, 64, torch.bfloat16)
    small = case(52, 3, 300, 2, 2, 128, 16, torch.bfloat16)
    both_ways(*big, 512, 64)
    both_ways(*small, 320, 64)
    both_ways(*small, 320, 128)
    both_ways(*big, 512, 64)


def test_other_dtypes_and_the_single_split_launch():
    both_ways(*case(53, 5, 1000, 2, 4, 64, 32, torch.float32), 1024, 256)
    both_ways(*case(54, 5, 200, 2, 1, 128, 16, torch.float16), 256, 256)  # one split: no scratch at all


def test_a_launch_beyond_the_array_is_refused():
    st, q, pos, bidx = case(55, 2, 100, 1, 1, 64, 16, torch.bfloat16)
    pk, pv = st.pool_planes()
    B, Hq, D, ctx, split = 4096, 32, 128, 8192, 64
    assert ops.decode_workspace_bytes(B, Hq, D, ctx, split) > _native.NOALLOC_SCRATCH_BYTES
    qq = torch.zeros((B, Hq, 1, D), dtype=torch.bfloat16, device=DEV)
    out, lse = torch.zeros_like(qq), torch.zeros((B, Hq, 1), dtype=torch.float32, device=DEV)
    pp = torch.zeros(B, dtype=torch.int32, device=DEV)
    bb = torch.zeros(B, dtype=torch.int64, device=DEV)
    pool = torch.zeros((Hq, 128, D), dtype=torch.bfloat16, device=DEV)
    table = torch.zeros((4, 8192 // 16), dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="the library's array holds"):
        ops.paged_decode_noalloc(qq, pool, pool, table, bb, pp, 16, ctx, out, lse, split_tokens=split)


def test_captured_in_a_graph_after_a_first_call_outside():
    """The first call on a device resolves the array's address and belongs outside a capture; after it the
    entry point is captured like any other: three replays with other positions and queries in between, each
    bit-identical to fp_paged_decode run eagerly on the same inputs."""
    st, q, pos, bidx = case(56, 9, 700, 4, 2, 128, 32, torch.bfloat16)
    pk, pv = st.pool_planes()
    lens = pos + 1
    out = torch.empty_like(q)
    lse = torch.empty((q.shape[0], q.shape[1], 1), dtype=torch.float32, device=DEV)
    run = lambda: ops.paged_decode_noalloc(q, pk, pv, st.cache.page_table, bidx, pos, st.P, 704, out, lse, split_tokens=128)
    run()  # outside the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run()
    for i in range(3):
        pos.copy_(torch.clamp(lens - 1 - 37 * i, min=0))
        q.copy_(randn(st.gen, tuple(q.shape), torch.bfloat16).to(DEV))
        g.replay()
        torch.cuda.synchronize()
        ref_out, ref_lse = ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, 704, split_tokens=128)
        assert torch.equal(out, ref_out) and torch.equal(lse, ref_lse), i
