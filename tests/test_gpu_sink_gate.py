"""GPU parity: the attention-sink gate (reference: Attention._post_attention, model.py:122-128)
fused into the decode merge / direct store and into the prefill epilogue.

The ungated kernel output is the attention result rounded to the model dtype, exactly what the
reference's gate receives; the oracle's gate applied to it must reproduce the fused kernel's
output up to the last bit of the dtype (the sigmoid is evaluated with a fast exp on the device).
"""

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, f64, randn

pytestmark = pytest.mark.gpu

NAME = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}
ULP = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2e-6}  # one step of the dtype, relative


def check_gated(gated, plain, lse, sinks, dtype):
    want = O.sink_gate(plain.float().cpu().numpy(), lse.float().cpu().numpy(), sinks.cpu().numpy(), NAME[dtype])
    got = gated.float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=ULP[dtype], atol=1e-30)
    if dtype != torch.float32:
        assert (got == want).mean() > 0.9  # a differing last bit is the exception


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("split", [64, 4096], ids=["merge-pass", "single-split"])
def test_decode_gate(dtype, split):
    st = PagedState(21, n_pages=80, page_size=16, max_batch=8, Hc=2, D=128, dtype=dtype)
    lens = [1, 17, 300, 64, 511]
    for L in lens:
        st.add_sequence(L)
    st.prefill_random()
    B, Hq = len(lens), 4
    q = randn(st.gen, (B, Hq, 1, 128), dtype).to(DEV)
    pos = torch.tensor([L - 1 for L in lens], dtype=torch.int32, device=DEV)
    pos[1] = -1  # a sequence without a visible key: lse = -inf, the gate must give 0, not NaN
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    sinks = (torch.randn(Hq, generator=st.gen) * 3).to(DEV)
    pk, pv = st.pool_planes()
    args = (q, pk, pv, st.cache.page_table, bidx, pos, st.P, 512)
    plain, lse0 = ops.paged_decode(*args, split_tokens=split)
    gated, lse1 = ops.paged_decode(*args, split_tokens=split, sinks=sinks)
    assert torch.equal(lse0, lse1)  # lse is returned ungated
    assert not gated[1].any() and not torch.isnan(gated).any()
    check_gated(gated, plain, lse0, sinks, dtype)
    # the row layout the output projection takes: [B, 1, Hq * D] through the stride arguments
    flat = torch.empty((B, 1, Hq * 128), dtype=dtype, device=DEV)
    ops.paged_decode(*args, split_tokens=split, sinks=sinks, out=flat.view(B, 1, Hq, 128).permute(0, 2, 1, 3))
    assert torch.equal(flat, gated.permute(0, 2, 1, 3).reshape(B, 1, Hq * 128))


def test_decode_gate_with_fused_append():
    dtype = torch.bfloat16
    outs = []
    for gate in (False, True):
        st = PagedState(22, n_pages=40, page_size=32, max_batch=6, Hc=2, D=128, dtype=dtype)
        lens = [0, 31, 32, 200]
        for L in lens:
            st.add_sequence(L + 1)
        st.lens = lens
        st.prefill_random()
        B = len(lens)
        k1, v1 = randn(st.gen, (B, 2, 1, 128), dtype).to(DEV), randn(st.gen, (B, 2, 1, 128), dtype).to(DEV)
        q = randn(st.gen, (B, 4, 1, 128), dtype).to(DEV)
        sinks = (torch.randn(4, generator=st.gen) * 2).to(DEV)
        pos = torch.tensor(lens, dtype=torch.int32, device=DEV)
        bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
        pk, pv = st.pool_planes()
        outs.append(ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, 256, split_tokens=64,
                                     k_new=k1, v_new=v1, sinks=sinks if gate else None) + (sinks,))
    assert torch.equal(outs[0][1], outs[1][1])
    check_gated(outs[1][0], outs[0][0], outs[0][1], outs[1][2], dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=str)
def test_prefill_gate(dtype):
    st = PagedState(23, n_pages=24, page_size=32, max_batch=4, Hc=2, D=128, dtype=dtype)
    b = st.add_sequence(300)
    st.prefill_random()
    Hq, Lq = 4, 300
    q = randn(st.gen, (1, Hq, Lq, 128), dtype).to(DEV)
    lim = torch.arange(1, Lq + 1, dtype=torch.int32)
    lim[:3] = 0  # rows without a visible key
    lim[100:200] = 200  # a bidirectional span
    bidx = torch.full((Lq,), b, dtype=torch.int64, device=DEV)
    sinks = (torch.randn(Hq, generator=st.gen) * 3).to(DEV)
    pk, pv = st.pool_planes()
    args = (q, pk, pv, st.cache.page_table, bidx, lim.to(DEV), st.P)
    plain, lse0 = ops.paged_prefill(*args)
    gated, lse1 = ops.paged_prefill(*args, sinks=sinks)
    assert torch.equal(lse0, lse1)
    assert not gated[:, :, :3].any() and not torch.isnan(gated).any()
    check_gated(gated, plain, lse0, sinks, dtype)


def test_sinks_argument_is_validated():
    st = PagedState(24, n_pages=8, page_size=16, max_batch=2, Hc=1, D=64, dtype=torch.bfloat16)
    st.add_sequence(20)
    st.prefill_random()
    q = randn(st.gen, (1, 2, 1, 64), torch.bfloat16).to(DEV)
    pk, pv = st.pool_planes()
    bidx = torch.tensor(st.slots, dtype=torch.int64, device=DEV)
    pos = torch.tensor([19], dtype=torch.int32, device=DEV)
    for bad in (torch.zeros(3, device=DEV), torch.zeros(2, device=DEV, dtype=torch.bfloat16), torch.zeros(2)):
        with pytest.raises(RuntimeError):
            ops.paged_decode(q, pk, pv, st.cache.page_table, bidx, pos, st.P, 32, sinks=bad)
