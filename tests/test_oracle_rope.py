"""Pins of the oracle's QK-norm + 3D rotary restatement (reference: model.py:105-120, rope.py:31-108).

The comparisons below evaluate the published formulation with torch library routines
(F.rms_norm, view_as_complex multiplication, repeat_interleave); nothing is imported from the
reference."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import paged_kv_oracle as O

DT = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}
EPS = float(torch.finfo(torch.float32).eps)  # what F.rms_norm(eps=None) uses, also for 16-bit inputs
STEP = {"bf16": 2.0 ** -7, "f16": 2.0 ** -10, "f32": 2e-6}


def make(seed, B, S, Hq, Hkv, D, name, with_2d=True):
    g = torch.Generator().manual_seed(seed)
    dt = DT[name]
    xq = (torch.randn(B, S, Hq, D, generator=g) * 2).to(dt)
    xk = (torch.randn(B, S, Hkv, D, generator=g) * 2).to(dt)
    xv = torch.randn(B, S, Hkv, D, generator=g).to(dt)
    ang = torch.rand(B, S, D // 4, generator=g) * 2 * math.pi
    f1 = torch.polar(torch.ones_like(ang), ang)
    f2 = None
    if with_2d:
        ang2 = torch.randn(B, S, Hq, D // 4, generator=g) * 3
        ang2[:, ::2] = 0  # text tokens: identity rotation (rope.py:63-64)
        f2 = torch.polar(torch.ones_like(ang2), ang2)
    return xq, xk, xv, f1, f2


@pytest.mark.parametrize("name", ["bf16", "f16", "f32"])
def test_rms_norm_rows_equals_torch(name):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(5, 7, 3, 128, generator=g) * 3).to(DT[name])
    want = F.rms_norm(x, (128,)).float().numpy()
    got = O.rms_norm_rows(x.float().numpy(), EPS, name)
    assert not np.array_equal(O.rms_norm_rows(x.float().numpy(), 2.0 ** -7, name), want)  # the dtype's own epsilon is not it
    np.testing.assert_allclose(got, want, rtol=STEP[name], atol=1e-30)
    if name != "f32":
        assert (got == want).mean() > 0.99
    # unit root-mean-square (up to eps and rounding)
    rms = np.sqrt((got.astype(np.float64) ** 2).mean(-1))
    assert np.allclose(rms, 1.0, atol={"bf16": 8e-3, "f16": 2e-3, "f32": 1e-5}[name])


@pytest.mark.parametrize("name", ["bf16", "f32"])
def test_rotary_equals_complex_multiplication(name):
    xq, _, _, f1, f2 = make(2, 2, 6, 4, 2, 64, name)
    x = xq.float()
    half = 32
    xt = torch.view_as_complex(x[..., :half].reshape(2, 6, 4, -1, 2))
    xh = torch.view_as_complex(x[..., half:].reshape(2, 6, 4, -1, 2))
    want = torch.cat([torch.view_as_real(xt * f1[:, :, None, :]).flatten(3),
                      torch.view_as_real(xh * f2).flatten(3)], -1).to(DT[name]).float().numpy()
    got = O.rotary_3d(x.numpy(), f1.numpy(), f2.numpy(), name)
    np.testing.assert_allclose(got, want, rtol=STEP[name], atol=1e-6)
    if name != "f32":
        assert (got == want).mean() > 0.99
    # without 2D angles the second half passes through
    got1 = O.rotary_3d(x.numpy(), f1.numpy(), None, name)
    assert np.array_equal(got1[..., half:], x.numpy()[..., half:]) and np.array_equal(got1[..., :half], got[..., :half])


def test_rotary_closed_forms():
    x = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 1, 16)
    zero = np.ones((1, 1, 4), dtype=np.complex64)
    assert np.array_equal(O.rotary_3d(x, zero, zero[:, :, None, :], "f32"), x)
    quarter = np.full((1, 1, 4), 1j, dtype=np.complex64)
    got = O.rotary_3d(x, quarter, quarter[:, :, None, :], "f32")[0, 0, 0]
    want = np.empty(16, dtype=np.float32)
    want[0::2] = -x[0, 0, 0, 1::2]  # (a, b) -> (-b, a)
    want[1::2] = x[0, 0, 0, 0::2]
    assert np.allclose(got, want, atol=1e-6)
    # first and second half use different angle tables: swapping them must change the result
    ang = np.exp(1j * np.linspace(0.1, 1.0, 4)).astype(np.complex64)[None, None]
    a = O.rotary_3d(x, ang, zero[:, :, None, :], "f32")
    b = O.rotary_3d(x, zero, ang[:, :, None, :], "f32")
    assert np.array_equal(a[..., 8:], x[..., 8:]) and np.array_equal(b[..., :8], x[..., :8]) and not np.allclose(a, b)
    # rotations keep the length of every pair
    y = O.rotary_3d(x, ang, ang[:, :, None, :], "f32")
    assert np.allclose(y[..., 0::2] ** 2 + y[..., 1::2] ** 2, x[..., 0::2] ** 2 + x[..., 1::2] ** 2, rtol=1e-5)


@pytest.mark.parametrize("name", ["bf16", "f32"])
def test_pre_attention_tail_equals_the_torch_composition(name):
    B, S, Hq, Hkv, D = 1, 9, 4, 2, 64
    xq, xk, xv, f1, f2 = make(3, B, S, Hq, Hkv, D, name)
    n_rep = Hq // Hkv
    q = F.rms_norm(xq, (D,))
    k = F.rms_norm(xk, (D,)).repeat_interleave(n_rep, dim=2)
    v = xv.repeat_interleave(n_rep, dim=2)

    def rot(x):
        xf = x.float()
        t = torch.view_as_complex(xf[..., : D // 2].reshape(B, S, Hq, -1, 2)) * f1[:, :, None, :]
        h = torch.view_as_complex(xf[..., D // 2:].reshape(B, S, Hq, -1, 2)) * f2
        return torch.cat([torch.view_as_real(t).flatten(3), torch.view_as_real(h).flatten(3)], -1).to(x.dtype)

    want = [rot(q).permute(0, 2, 1, 3), rot(k).permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)]
    got = O.pre_attention_tail(xq.float().numpy(), xk.float().numpy(), xv.float().numpy(), f1.numpy(), f2.numpy(),
                               n_rep, name, EPS)
    for g_, w in zip(got, want):
        np.testing.assert_allclose(g_, w.float().numpy(), rtol=2 * STEP[name], atol=1e-6)
    assert np.array_equal(got[2], want[2].float().numpy())
    # replicas of one K head differ only through the per-head 2D angles
    kk = got[1]
    assert np.array_equal(kk[:, 0, :, : D // 2], kk[:, 1, :, : D // 2]) and not np.array_equal(kk[:, 0], kk[:, 1])
