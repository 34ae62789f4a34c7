"""GPU parity: QK norm + 3D rotary embedding + cache insert in one launch against the oracle's
restatement of model.py:110-119 followed by the oracle's append.

Floating point: the kernel and the oracle round at the same two places (after the norm, after the
rotation); what is left is the order of the fp32 sum of squares and fused multiply-adds, so results
agree to one step of the dtype and are identical almost everywhere.  V rows are copied: bit-exact.
"""

import math

import numpy as np
import pytest
import torch

from falcon_perception_amd import ops
from oracle import paged_kv_oracle as O
from tests.gpu_cases import DEV, PagedState, bits, f64

pytestmark = pytest.mark.gpu

NAME = {torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32"}
STEP = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 4e-6}
EPS = float(torch.finfo(torch.float32).eps)


def inputs(gen, B, S, Hq, Hkv, D, dtype, with_2d):
    # one projection output, sliced like model.py:106-109 (strided views, no copies)
    qkv = (torch.randn(B, S, (Hq + 2 * Hkv) * D, generator=gen) * 2).to(dtype)
    xq, xk, xv = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
    xq, xk, xv = xq.view(B, S, Hq, D), xk.view(B, S, Hkv, D), xv.view(B, S, Hkv, D)
    ang = torch.rand(B, S, D // 4, generator=gen) * 2 * math.pi
    f1 = torch.polar(torch.ones_like(ang), ang)
    f2 = None
    if with_2d:
        ang2 = torch.randn(B, S, Hq, D // 4, generator=gen) * 3
        ang2[:, ::3] = 0  # text tokens rotate by zero
        f2 = torch.polar(torch.ones_like(ang2), ang2)
    return qkv, xq, xk, xv, f1, f2


def close(got, want, dtype):
    got, want = got.float().cpu().numpy(), np.asarray(want, dtype=np.float32)
    # a last-bit difference of a normalised value (magnitude up to ~4) passes through the rotation as an
    # absolute error, also into outputs that are small by cancellation: absolute bound of one such step
    np.testing.assert_allclose(got, want, rtol=STEP[dtype], atol=4 * STEP[dtype])
    if dtype != torch.float32:
        assert (got == want).mean() > 0.98


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("D,Hq,Hkv", [(128, 4, 2), (64, 8, 8), (128, 6, 2), (128, 8, 2), (64, 8, 1), (128, 16, 8)])
def test_prefill_step(dtype, D, Hq, Hkv):
    prefill_step(dtype, D, Hq, Hkv)


@pytest.mark.parametrize("dtype,D,Hq,Hkv", [(torch.bfloat16, 32, 4, 2), (torch.bfloat16, 256, 4, 2), (torch.bfloat16, 512, 2, 1),
                                            (torch.float32, 16, 4, 2), (torch.float32, 256, 2, 2), (torch.float16, 32, 2, 2),
                                            (torch.float16, 256, 3, 1)], ids=str)
def test_prefill_step_at_other_head_dims(dtype, D, Hq, Hkv):
    """Rows of 4 to 64 sixteen-byte vectors: every lane-group width of the two kernels."""
    prefill_step(dtype, D, Hq, Hkv)


def prefill_step(dtype, D, Hq, Hkv):
    P = 16
    st = PagedState(31, n_pages=64, page_size=P, max_batch=6, Hc=Hq, D=D, dtype=dtype)
    lens = [37, 150, 64]
    slots = [st.add_sequence(L) for L in lens]
    bidx = np.concatenate([np.full(L, b) for b, L in zip(slots, lens)] + [np.zeros(5, dtype=np.int64)])  # + padding rows
    pos = np.concatenate([np.arange(L) for L in lens] + [np.zeros(5, dtype=np.int64)])
    Lp = len(bidx)
    qkv, xq, xk, xv, f1, f2 = inputs(st.gen, 1, Lp, Hq, Hkv, D, dtype, True)
    cache = st.cache
    before = cache.kv_cache.clone()
    q, K, V = cache.insert_qkv_norm_rope(0, xq.to(DEV), xk.to(DEV), xv.to(DEV), f1.to(DEV), f2.to(DEV),
                                         input_pos=torch.from_numpy(pos)[None].to(DEV),
                                         batch_idx=torch.from_numpy(bidx)[None].to(DEV))
    eq, ek, ev = O.pre_attention_tail(xq.float().numpy(), xk.float().numpy(), xv.float().numpy(), f1.numpy(),
                                      f2.numpy(), Hq // Hkv, NAME[dtype], EPS)
    close(q, eq, dtype)
    assert q.shape == (1, Hq, Lp, D) and K.shape == (1, Hq, st.cache.n_pages * P, D)
    # expected pool: the oracle's append of the oracle's rotated rows
    pool = before.float().cpu().numpy()
    want = pool.copy()
    O.append_prefill(want, 0, ek, ev, st.mirror.page_table, bidx[None], pos[None], P)
    got = cache.kv_cache.float().cpu().numpy()
    live = np.ones(got.shape[4], dtype=bool)
    live[0] = False  # slot 0 takes the padding rows: unspecified
    close(torch.from_numpy(got[0, 0, 0][:, live]), want[0, 0, 0][:, live], dtype)
    assert np.array_equal(got[0, 1, 0][:, live], want[0, 1, 0][:, live])  # V: copies
    # slots no token maps to keep their bits
    touched = np.zeros(got.shape[4], dtype=bool)
    touched[O.prefill_slots(st.mirror.page_table, bidx[None], pos[None], P, got.shape[4]).reshape(-1)] = True
    assert np.array_equal(bits(cache.kv_cache[0, :, 0][:, :, ~torch.from_numpy(touched)]),
                          bits(before[0, :, 0][:, :, ~torch.from_numpy(touched)]))


@pytest.mark.parametrize("with_2d", [True, False], ids=["golden-2d", "1d-only"])
def test_decode_step(with_2d):
    dtype, D, Hkv, P = torch.bfloat16, 128, 2, 32
    Hq = 4
    H_pool = Hq if with_2d else Hkv  # without per-head angles the cache may keep the kv heads only
    st = PagedState(32, n_pages=48, page_size=P, max_batch=9, Hc=H_pool, D=D, dtype=dtype)
    lens = [0, 31, 32, 100, 255]
    for L in lens:
        st.add_sequence(L + 1)
    B = len(lens)
    qkv, xq, xk, xv, f1, f2 = inputs(st.gen, B, 1, Hq, Hkv, D, dtype, with_2d)
    bidx = torch.tensor(st.slots, dtype=torch.int64)
    bidx_pad = torch.cat([bidx, torch.tensor([0])])  # a graph-padding row: batch slot 0, unmapped -> page 0
    pos = torch.tensor(lens, dtype=torch.int32).view(B, 1)
    before = st.cache.kv_cache.clone()
    q, K, V = st.cache.insert_qkv_norm_rope(0, xq.to(DEV), xk.to(DEV), xv.to(DEV), f1.to(DEV),
                                            f2.to(DEV) if with_2d else None, input_pos=pos.to(DEV), batch_idx=bidx.to(DEV))
    del bidx_pad
    eq, ek, ev = O.pre_attention_tail(xq.float().numpy(), xk.float().numpy(), xv.float().numpy(), f1.numpy(),
                                      f2.numpy() if with_2d else None, H_pool // Hkv, NAME[dtype], EPS)
    if not with_2d:  # q has Hq heads, K only the kv heads
        eq = O.pre_attention_tail(xq.float().numpy(), xk.float().numpy(), xv.float().numpy(), f1.numpy(), None,
                                  1, NAME[dtype], EPS)[0]
    close(q, eq, dtype)
    pool = before.float().cpu().numpy()
    want = pool.copy()
    O.append_decode(want, 0, ek, ev, st.mirror.page_table, bidx.numpy(), pos.numpy(), P)
    got = st.cache.kv_cache.float().cpu().numpy()
    close(torch.from_numpy(got[0, 0, 0]), want[0, 0, 0], dtype)
    assert np.array_equal(got[0, 1, 0], want[0, 1, 0])
    # and the attention that follows sees the new token: fused decode over the pool equals the oracle on the oracle's pool
    out, lse = ops.paged_decode(q, K[0], V[0], st.cache.page_table, bidx.to(DEV), pos.view(-1).to(DEV), P, 256)
    eo, el = O.decode_attention(eq.astype(np.float64), want[0, 0, 0].astype(np.float64), want[0, 1, 0].astype(np.float64),
                                st.mirror.page_table, st.slots, pos.view(-1).numpy(), P)
    np.testing.assert_allclose(f64(out), eo, atol=3e-2, rtol=2e-2)


def test_arguments_are_validated():
    st = PagedState(33, n_pages=8, page_size=16, max_batch=3, Hc=2, D=64, dtype=torch.bfloat16)
    b = st.add_sequence(10)
    qkv, xq, xk, xv, f1, f2 = inputs(st.gen, 1, 10, 4, 2, 64, torch.bfloat16, True)
    pk, pv = st.pool_planes()
    args = dict(page_size=16)
    bidx = torch.full((10,), b, dtype=torch.int64, device=DEV)
    pos = torch.arange(10, device=DEV)
    with pytest.raises(RuntimeError, match="one cached K head per query head"):
        ops.qkv_norm_rope_append(xq.to(DEV), xk.to(DEV), xv.to(DEV), f1.to(DEV), f2.to(DEV), pk, pv,
                                 st.cache.page_table, bidx, pos, 16)
    with pytest.raises(RuntimeError, match="complex64"):
        ops.qkv_norm_rope_append(xq.to(DEV), xk.to(DEV), xv.to(DEV), torch.view_as_real(f1).to(DEV), None, pk, pv,
                                 st.cache.page_table, bidx, pos, 16)
    del args
