"""Pins the CPU oracle's conv restatement (no GPU): closed forms, a library routine on
dequantised values, the forward/update invariant, and the rounding and exp primitives."""
import ctypes as C

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from quamba_amd import synth


def test_exp_matches_libm_within_2ulp():
    g = np.random.default_rng(0)
    x = np.concatenate([g.uniform(-87, 88, 20000), g.uniform(-2, 2, 20000), np.array([0.0, -0.0, 1.0, -1.0])])
    x = x.astype(np.float32)
    got = oracle.expf(x).astype(np.float64)
    want = np.exp(x.astype(np.float64))
    ulp = np.spacing(want.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - want) / ulp) < 2.0
    assert oracle.expf(np.float32([89.0]))[0] == np.inf
    assert oracle.expf(np.float32([-88.0]))[0] == 0.0
    assert oracle.expf(np.float32([0.0]))[0] == 1.0


def test_rounding_primitives_on_half_grid():
    l = oracle.lib()
    for v, away, even in [(0.5, 1, 0), (1.5, 2, 2), (2.5, 3, 2), (-0.5, -1, 0), (-1.5, -2, -2), (-2.5, -3, -2),
                          (126.5, 127, 126), (127.5, 127, 127), (-128.5, -128, -128), (300.0, 127, 127),
                          (-300.0, -128, -128), (0.49999997, 0, 0)]:
        assert l.qo_sat8_half_away(C.c_float(v)) == away
        assert l.qo_sat8_rne(C.c_float(v)) == even


@pytest.mark.parametrize("width", [2, 3, 4])
def test_unit_taps_give_sliding_window_sum(width):
    g = np.random.default_rng(width)
    x = g.integers(-20, 21, (2, 3, 37)).astype(np.int8)
    w = np.ones((3, width), np.int8)
    out = oracle.conv1d_fwd(x, w, None, 1.0, 1.0, 1.0, 1.0, silu=False)
    xp = np.pad(x.astype(np.int64), ((0, 0), (0, 0), (width - 1, 0)))
    want = sum(xp[:, :, j:j + 37] for j in range(width))
    np.testing.assert_array_equal(out, np.clip(want, -128, 127))


def test_single_tap_selects_the_right_lag():
    # taps e_j pick x[t-(k-1-j)]: a reversed or shifted tap order fails this
    x = np.arange(1, 11, dtype=np.int8).reshape(1, 1, 10)
    for k in (2, 3, 4):
        for j in range(k):
            w = np.zeros((1, k), np.int8)
            w[0, j] = 1
            out = oracle.conv1d_fwd(x, w, None, 1.0, 1.0, 1.0, 1.0, silu=False)
            lag = k - 1 - j
            want = np.concatenate([np.zeros(lag, np.int8), x[0, 0, :10 - lag]])
            np.testing.assert_array_equal(out[0, 0], want)


@pytest.mark.parametrize("tapwise", [False, True])
@pytest.mark.parametrize("silu", [False, True])
def test_against_torch_conv1d_on_dequantised_values(tapwise, silu):
    B, D, L, k = 2, 48, 129, 4
    qx, sx = synth.quantize_absmax(synth.activations((B, D, L), 1, 7, "x"))
    qw, sw, qb, sb = synth.conv_weights(D, k, 7)
    so = synth.conv_output_scale(qx, sx, qw, sw, qb, sb, silu)
    out = oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so, silu=silu, tapwise=tapwise)
    x = torch.from_numpy(qx.astype(np.float64) * float(sx))
    w = torch.from_numpy(qw.astype(np.float64) * float(sw)).unsqueeze(1)
    b = torch.from_numpy(qb.astype(np.float64) * float(sb))
    ref = F.conv1d(x, w, b, padding=k - 1, groups=D)[..., :L]
    if silu:
        ref = F.silu(ref)
    y = (ref / float(so)).numpy()
    want = np.clip(np.where(y >= 0, np.floor(y + 0.5), np.ceil(y - 0.5)), -128, 127)
    diff = np.abs(out.astype(np.int64) - want.astype(np.int64))
    assert diff.max() <= 1                     # fp32 vs fp64 can only move a value across a tie
    assert (diff != 0).mean() < 2e-3
    assert np.abs(out).max() >= 126            # the scale uses the full int8 range


def test_forward_equals_update_applied_step_by_step():
    B, D, L, k = 2, 16, 40, 4
    qx, sx = synth.quantize_absmax(synth.activations((B, D, L), 1, 3, "x"))
    qw, sw, qb, sb = synth.conv_weights(D, k, 3)
    so = synth.conv_output_scale(qx, sx, qw, sw, qb, sb)
    fwd = oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so, tapwise=True)   # same op order as update
    for slen in (k, k - 1):
        state = np.zeros((B, D, slen), np.int8)
        for t in range(L):
            o, state = oracle.conv1d_update(qx[:, :, t], state, qw, qb, sx, sw, sb, so)
            np.testing.assert_array_equal(o, fwd[:, :, t])
        np.testing.assert_array_equal(state[:, :, -(k - 1):], qx[:, :, L - (k - 1):])
    # the sum-first order of the seqlen-contiguous kernel may differ by one step at ties only
    fwd2 = oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so, tapwise=False)
    assert np.abs(fwd2.astype(int) - fwd.astype(int)).max() <= 1


def test_no_bias_and_saturation():
    x = np.full((1, 2, 8), 127, np.int8)
    w = np.full((2, 4), 127, np.int8)
    out = oracle.conv1d_fwd(x, w, None, 1.0, 1.0, 1.0, 1.0, silu=False)
    assert (out == 127).all()
    out = oracle.conv1d_fwd(x, (-w).astype(np.int8), None, 1.0, 1.0, 1.0, 1.0, silu=False)
    assert (out == -128).all()
    out = oracle.conv1d_fwd(np.zeros((1, 2, 0), np.int8), w, None, 1.0, 1.0, 1.0, 1.0)
    assert out.shape == (1, 2, 0)
