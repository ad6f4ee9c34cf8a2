"""Pins the CPU oracle's gated RMS norm (no GPU) against torch's own ops in float64 and against invariants."""
import numpy as np
import pytest
import torch

import oracle


def _inputs(M=5, N=256, seed=0):
    g = np.random.default_rng(seed)
    x = (g.standard_normal((M, N)) * 3).astype(np.float16)
    w = (1 + 0.2 * g.standard_normal(N)).astype(np.float16)
    qz = g.integers(-128, 128, (M, N)).astype(np.int8)
    return x, w, qz


@pytest.mark.parametrize("norm_before_gate", [True, False])
@pytest.mark.parametrize("group_size", [None, 64])
def test_matches_torch_in_float64(norm_before_gate, group_size):
    x, w, qz = _inputs()
    y, _, _ = oracle.rmsnorm_gated(x, w, qz, eps=1e-5, z_scale=0.03, group_size=group_size, norm_before_gate=norm_before_gate)
    xt = torch.from_numpy(x).double()
    z = torch.from_numpy(qz).double() * float(np.float32(0.03))
    gate = torch.nn.functional.silu(z)
    if not norm_before_gate:
        xt = xt * gate
    g = x.shape[1] if group_size is None else group_size
    xg = xt.reshape(x.shape[0], -1, g)
    want = (xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + float(np.float32(1e-5)))).reshape(x.shape) * torch.from_numpy(w).double()
    if norm_before_gate:
        want = want * gate
    np.testing.assert_allclose(y, want.numpy(), rtol=1e-12, atol=1e-12)


def test_unit_weight_rows_have_unit_rms_and_scale_invariance():
    x, w, _ = _inputs(seed=2)
    y, _, _ = oracle.rmsnorm_gated(x, np.ones_like(w), eps=0.0)
    np.testing.assert_allclose(np.sqrt((y * y).mean(axis=1)), 1.0, rtol=1e-12)
    y2, _, _ = oracle.rmsnorm_gated((x.astype(np.float32) * 2).astype(np.float16), np.ones_like(w), eps=0.0)
    np.testing.assert_allclose(y2, y, rtol=1e-12)              # doubling fp16 values is exact


def test_output_modes():
    x, w, qz = _inputs(seed=3)
    y, q, _ = oracle.rmsnorm_gated(x, w, qz, eps=1e-5, z_scale=0.02, out_mode="static", out_scale=0.05)
    assert q.dtype == np.int8 and np.max(np.abs(q.astype(np.float64) * float(np.float32(0.05)) - np.clip(y, -6.4, 6.35))) <= 0.0251
    y, q, s = oracle.rmsnorm_gated(x, w, qz, eps=1e-5, z_scale=0.02, group_size=64, out_mode="dynamic")
    assert s.shape == (4, 5)
    np.testing.assert_allclose(s.T, y.reshape(5, 4, 64).max(axis=2) / 127, rtol=1e-6)
    assert q.reshape(5, 4, 64).max(axis=2).min() == 127          # the largest entry of every group maps to 127
