"""GPU: chunked-prefill launches too small for the GPU are also cut along the keys (several workgroups
share a query tile, a merge pass combines their partial results).  The cut changes the order of the
additions only: results stay within the dtype's tolerance of the oracle and of the uncut launch."""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, f64, randn

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: (2e-2, 1e-2), torch.float16: (4e-3, 4e-3), torch.float32: (2e-5, 2e-5)}


def make_case(dtype, D, G, P, lens, pads, seed=31):
    Hc = 2
    st = PagedState(seed, n_pages=sum(-(-n // P) for n in lens) + 4, page_size=P, max_batch=len(lens) + 2, Hc=Hc, D=D,
                    dtype=dtype)
    bidx, pos = [], []
    for n, pad in zip(lens, pads):
        b = st.add_sequence(n)
        bidx += [b] * n + [0] * pad
        pos += list(range(n)) + [0] * pad
    Lq = len(bidx)
    bidx_t = torch.tensor(bidx, dtype=torch.int64)[None].to(DEV)
    pos_t = torch.tensor(pos, dtype=torch.int64)[None].to(DEV)
    k = randn(st.gen, (1, Hc, Lq, D), dtype)
    v = randn(st.gen, (1, Hc, Lq, D), dtype)
    q = randn(st.gen, (1, Hc * G, Lq, D), dtype)
    st.cache.insert_kv(0, k.to(DEV), v.to(DEV), input_pos=pos_t, batch_idx=bidx_t)
    lim = (pos_t.view(-1) + 1).to(torch.int32)
    lim[bidx_t.view(-1) == 0] = 0
    return st, q, bidx_t.view(-1), lim


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D,G,P", [(128, 2, 128), (64, 4, 16), (128, 1, 64), (128, 8, 32)])
def test_key_shares_match_the_oracle_and_the_uncut_launch(dtype, D, G, P):
    # several sequences in one 128-row tile, one of them shorter than the number of shares in tiles
    st, q, bidx, lim = make_case(dtype, D, G, P, lens=[700, 40, 3, 300], pads=[3, 0, 5, 1])
    pk, pv = st.pool_planes()
    Hq, Hc, Lq = q.shape[1], pk.shape[0], q.shape[2]
    need = ops.prefill_workspace_bytes(Lq, Hq, Hc, D, dtype)
    assert need > 0  # a launch of a few workgroups: the library wants to cut it
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    out0, lse0 = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, workspace=False)
    out1, lse1 = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, workspace=ws)
    out2, lse2 = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P)  # allocates its own
    assert torch.equal(out1, out2) and torch.equal(lse1, lse2)
    atol, rtol = TOL[dtype]
    eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, bidx.cpu().numpy(), None,
                                       lim.cpu().numpy(), P)
    for out, lse in ((out0, lse0), (out1, lse1)):
        np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
        np.testing.assert_allclose(f64(lse), el, atol=max(atol * 0.1, 1e-4), rtol=rtol)
    pad = (bidx == 0).cpu().numpy()
    assert not f64(out1)[:, :, pad].any() and np.isneginf(f64(lse1)[:, :, pad]).all()


def test_a_smaller_workspace_gives_a_coarser_cut_and_the_same_answer():
    dtype, D, P = torch.bfloat16, 128, 128
    st, q, bidx, lim = make_case(dtype, D, 2, P, lens=[900], pads=[0])
    pk, pv = st.pool_planes()
    Hq, Lq = q.shape[1], q.shape[2]
    need = ops.prefill_workspace_bytes(Lq, Hq, pk.shape[0], D, dtype)
    two_shares = 2 * Lq * Hq * (D * 2 + 8)  # per row and head: D bf16 results, maximum and denominator
    assert need > two_shares
    full, _ = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P,
                                workspace=torch.empty(need, dtype=torch.uint8, device=DEV))
    for nbytes in (two_shares, two_shares - 16, 16):  # two shares, then none
        out, _ = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P,
                                   workspace=torch.empty(nbytes, dtype=torch.uint8, device=DEV))
        np.testing.assert_allclose(f64(out), f64(full), atol=2e-2, rtol=1e-2)
    uncut, _ = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, workspace=False)
    tiny, _ = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P,
                                workspace=torch.empty(16, dtype=torch.uint8, device=DEV))
    assert torch.equal(uncut, tiny)  # a workspace that holds no second share: the one-launch path


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
def test_sink_gate_through_the_merge_pass(dtype):
    D, P = 128, 64
    st, q, bidx, lim = make_case(dtype, D, 2, P, lens=[500, 120], pads=[4, 0])
    pk, pv = st.pool_planes()
    sinks = torch.linspace(-3.0, 3.0, q.shape[1], device=DEV)
    cut, lse_c = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, sinks=sinks)
    one, lse_o = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, sinks=sinks, workspace=False)
    atol, rtol = TOL[dtype]
    np.testing.assert_allclose(f64(cut), f64(one), atol=atol, rtol=rtol)
    np.testing.assert_allclose(f64(lse_c), f64(lse_o), atol=max(atol * 0.1, 1e-5), rtol=rtol)


def test_large_launches_ask_for_no_workspace():
    assert ops.prefill_workspace_bytes(23040, 16, 8, 128, torch.bfloat16) == 0
    assert ops.prefill_workspace_bytes(23040, 16, 8, 128, torch.float32) == 0
    assert ops.prefill_workspace_bytes(512, 16, 8, 128, torch.float32) == 8 * 512 * 16 * 130 * 4
    # fp32 is still cut at about one workgroup per CU, where the faster 16-bit kernels no longer are
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rows = 128 * (cus // 8)
    assert ops.prefill_workspace_bytes(rows, 16, 8, 128, torch.bfloat16) == 0
    assert ops.prefill_workspace_bytes(rows, 16, 8, 128, torch.float32) == 4 * rows * 16 * 130 * 4
    assert ops.prefill_workspace_bytes(512, 16, 8, 128, torch.bfloat16) == 8 * 512 * 16 * (128 * 2 + 8)
    with pytest.raises(RuntimeError, match="fp_paged_prefill_workspace_bytes"):
        ops.prefill_workspace_bytes(512, 12, 8, 128, torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
def test_the_passes_stay_inside_the_workspace_they_asked_for(dtype):
    D, P = 128, 64
    st, q, bidx, lim = make_case(dtype, D, 2, P, lens=[333, 900, 70], pads=[1, 0, 2])
    pk, pv = st.pool_planes()
    need = ops.prefill_workspace_bytes(q.shape[2], q.shape[1], pk.shape[0], D, dtype)
    assert need > 0
    guard = 1 << 20
    for nbytes in (need, need // 2, need // 4 + 16):  # what the library asked for, and less (coarser cuts)
        buf = torch.full((nbytes + guard,), 0x5A, dtype=torch.uint8, device=DEV)
        out, lse = ops.paged_prefill(q.to(DEV), pk, pv, st.cache.page_table, bidx, lim, P, workspace=buf[:nbytes])
        assert bool((buf[nbytes:] == 0x5A).all())
        atol, rtol = TOL[dtype]
        eo, el = O.prefill_attention_paged(f64(q), f64(pk), f64(pv), st.mirror.page_table, bidx.cpu().numpy(), None,
                                           lim.cpu().numpy(), P)
        np.testing.assert_allclose(f64(out), eo, atol=atol, rtol=rtol)
