"""Pins of the oracle's post-attention sink gate (reference: model.py:122-128)."""
import numpy as np
import torch

from oracle import paged_kv_oracle as O


def test_round_to_dtype_equals_torch_casts():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 10.0 ** rng.integers(-6, 6, 4096),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 65504.0, 70000.0, 3.0e38, 1e-40,
                                  np.inf, -np.inf], dtype=np.float32)])
    t = torch.from_numpy(x)
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16), ("f32", torch.float32)):
        want = t.to(dt).float().numpy()
        got = O.round_to_dtype(x, name)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), name
    # ties go to even: 1 + 2^-8 is halfway between two bf16 values
    assert O.round_to_dtype(np.float32(1.00390625), "bf16") == np.float32(1.0)
    assert O.round_to_dtype(np.float32(1.01171875), "bf16") == np.float32(1.015625)
    assert np.isnan(O.round_to_dtype(np.float32(np.nan), "bf16"))


def test_sink_gate_equals_the_torch_expression():
    g = torch.Generator().manual_seed(3)
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16), ("f32", torch.float32)):
        out = torch.randn(3, 5, 2, 16, generator=g).to(dt)
        lse = torch.randn(3, 5, 2, generator=g) * 4
        sinks = (torch.randn(5, generator=g) * 3).to(dt)
        # the reference's lines, on library tensors
        want = (out * torch.sigmoid(lse - sinks.view(1, -1, 1)).unsqueeze(-1)).to(out.dtype)
        got = O.sink_gate(out.float().numpy(), lse.numpy(), sinks.float().numpy(), name)
        tol = {"bf16": 2 ** -7, "f16": 2 ** -10, "f32": 1e-6}[name]  # at most one rounding step apart
        assert np.allclose(got, want.float().numpy(), rtol=tol, atol=1e-7)
        if name != "f32":  # identical almost everywhere once rounded to 8 or 11 bits
            assert (got == want.float().numpy()).mean() > 0.98


def test_sink_gate_closed_forms():
    out = np.array([[[[1.0, -2.0, 0.5, 8.0]]]], dtype=np.float32)  # exactly representable everywhere
    lse = np.array([[[0.75]]], dtype=np.float32)
    assert np.array_equal(O.sink_gate(out, lse, [-1e30], "bf16"), out)              # sigmoid -> 1
    assert np.array_equal(O.sink_gate(out, lse, [0.75], "bf16"), out * 0.5)         # sink == lse
    assert np.array_equal(O.sink_gate(out, [[[-np.inf]]], [0.0], "bf16"), out * 0)  # no visible key
    big = O.sink_gate(out, lse, [1e30], "f32")
    assert np.array_equal(big, out * 0)
    # a dropped sign (sinks - lse) or a per-batch instead of per-head broadcast must fail
    out2 = np.ones((2, 3, 1, 4), dtype=np.float32)
    lse2 = np.zeros((2, 3, 1), dtype=np.float32)
    got = O.sink_gate(out2, lse2, [-2.0, 0.0, 2.0], "f32")
    want = 1.0 / (1.0 + np.exp(-np.array([2.0, 0.0, -2.0])))
    assert np.allclose(got[:, :, 0, 0], np.broadcast_to(want, (2, 3)), rtol=1e-6)
