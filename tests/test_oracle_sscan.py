"""Pins the CPU oracle's selective-scan restatement (no GPU): float64 brute force written from
the mathematics, closed forms, and the forward/update invariant."""
import numpy as np
import pytest

import oracle
from oracle import naive
from quamba_amd import synth


def _deq(d):
    f = lambda k, s: None if d[k] is None else d[k].astype(np.float64) * float(d[s])
    return dict(u=f("u", "s_u"), dt=f("dt", "s_dt"), B=f("B", "s_B"), C=f("C", "s_C"), z=f("z", "s_z"),
                A=-np.exp(f("A_log", "s_A")), D=f("D", "s_D"), db=f("dt_bias", "s_db"))


def _run(d, **kw):
    return oracle.sscan_fwd(d["u"], d["dt"], d["A_log"], d["B"], d["C"], d["D"], d["dt_bias"], d["z"],
                            s_u=d["s_u"], s_delta=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                            s_D=d["s_D"], s_db=d["s_db"], s_z=d["s_z"], **kw)


@pytest.mark.parametrize("with_z", [True, False])
def test_against_float64_brute_force(with_z):
    d = synth.mamba1_scan_inputs(2, 96, 24, 16, seed=3, with_z=with_z)
    y, st8, st32 = _run(d, s_state=0.01)
    r = _deq(d)
    y64, h64 = naive.selective_scan(r["u"], r["dt"], r["A"], r["B"], r["C"], r["D"], r["z"], r["db"])
    assert np.abs(y - y64).max() <= 1e-4 * max(1.0, np.abs(y64).max())
    assert np.abs(st32 - h64).max() <= 1e-5 * np.abs(h64).max()
    want8 = np.clip(np.where(st32 >= 0, np.floor(st32 / np.float32(0.01) + 0.5), np.ceil(st32 / np.float32(0.01) - 0.5)), -128, 127)
    assert np.abs(st8.astype(int) - want8.astype(int)).max() <= 1 and (st8 != want8).mean() < 0.01


def test_zero_step_size_leaves_only_the_skip_path():
    # dt == 0 without softplus: a = 1, b = 0, so h stays 0 and y = D u silu(z)
    d = synth.mamba1_scan_inputs(1, 20, 8, 16, seed=5)
    d["dt"] = np.zeros_like(d["dt"])
    d["dt_bias"] = None
    y, _, st32 = _run(d, softplus=False)
    r = _deq(d)
    want = (r["D"][None, :, None] * r["u"] * naive.silu(r["z"])).transpose(0, 2, 1)
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-6)
    assert (st32 == 0).all()


def test_constant_inputs_give_a_geometric_series():
    B_, D_, L, N = 1, 2, 50, 4
    one = lambda shape, v: np.full(shape, v, np.int8)
    A_log = np.zeros((D_, N), np.int8)          # A = -1
    s_dt, s_u, s_B, s_C = 0.01, 0.5, 0.25, 0.125
    y, _, st = oracle.sscan_fwd(one((B_, D_, L), 4), one((B_, D_, L), 10), A_log, one((B_, N, L), 8), one((B_, N, L), 16),
                                None, None, None, s_u=s_u, s_delta=s_dt, s_A=1.0, s_B=s_B, s_C=s_C, softplus=False)
    dt, u, Bv, Cv = 10 * s_dt, 4 * s_u, 8 * s_B, 16 * s_C
    a, b = np.exp(-dt), dt * Bv * u
    t = np.arange(1, L + 1)
    h = b * (1 - a ** t) / (1 - a)
    np.testing.assert_allclose(y[0, :, 0], N * h * Cv, rtol=2e-5)
    np.testing.assert_allclose(st[0, 0], np.full(N, h[-1]), rtol=2e-5)


def test_state_index_and_group_layout():
    # only state n=2 of B and n=2 of C non-zero -> output non-zero; mismatched n -> exactly zero
    B_, D_, L, N = 1, 3, 6, 4
    u = np.full((B_, D_, L), 10, np.int8)
    dt = np.full((B_, D_, L), 10, np.int8)
    A_log = np.zeros((D_, N), np.int8)
    Bm = np.zeros((B_, N, L), np.int8); Bm[:, 2] = 5
    Cm = np.zeros((B_, N, L), np.int8); Cm[:, 2] = 7
    kw = dict(s_u=1.0, s_delta=0.01, s_A=1.0, s_B=1.0, s_C=1.0, softplus=False)
    y, _, st = oracle.sscan_fwd(u, dt, A_log, Bm, Cm, None, None, None, **kw)
    assert (y > 0).all() and (st[:, :, 2] > 0).all() and (st[:, :, [0, 1, 3]] == 0).all()
    Cm2 = np.zeros_like(Cm); Cm2[:, 1] = 7
    y2, _, _ = oracle.sscan_fwd(u, dt, A_log, Bm, Cm2, None, None, None, **kw)
    assert (y2 == 0).all()
    # two B/C groups: channel d uses group d // (D/G)
    Bg = np.zeros((B_, 2, N, L), np.int8); Bg[:, 1, 0] = 5
    Cg = np.zeros((B_, 2, N, L), np.int8); Cg[:, 1, 0] = 7
    y3, _, _ = oracle.sscan_fwd(np.full((B_, 4, L), 10, np.int8), np.full((B_, 4, L), 10, np.int8),
                                np.zeros((4, N), np.int8), Bg, Cg, None, None, None, **kw)
    assert (y3[:, :, :2] == 0).all() and (y3[:, :, 2:] > 0).all()


def test_forward_equals_update_iterated_with_fp32_state():
    d = synth.mamba1_scan_inputs(2, 40, 12, 16, seed=9)
    y, _, st32 = _run(d)
    state = np.zeros((2, 12, 16), np.float32)
    for t in range(40):
        yt, state = oracle.sscan_update(state, d["u"][:, :, t], d["dt"][:, :, t], d["A_log"], d["B"][:, :, t],
                                        d["C"][:, :, t], d["D"], d["dt_bias"], d["z"][:, :, t],
                                        s_x=d["s_u"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                                        s_D=d["s_D"], s_db=d["s_db"], s_z=d["s_z"])
        np.testing.assert_allclose(yt, y[:, t], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(state, st32, rtol=1e-5, atol=1e-7)


def test_update_requantises_int8_state_half_to_even():
    # h = 0*dA + dB*x chosen so h/s lands exactly on .5: rint goes to the even neighbour
    x = np.array([[1]], np.int8); dt = np.array([[1]], np.int8)
    A_log = np.zeros((1, 2), np.int8)
    Bm = np.array([[1, 3]], np.int8); Cm = np.zeros((1, 2), np.int8)
    state = np.zeros((1, 1, 2), np.int8)
    _, st = oracle.sscan_update(state, x, dt, A_log, Bm, Cm, None, None, None, s_x=1.0, s_dt=1.0, s_A=1.0,
                                s_B=0.5, s_C=1.0, s_state=1.0, softplus=False)
    # h = (0.5*1*1, 1.5*1*1) -> rint -> (0, 2)
    np.testing.assert_array_equal(st[0, 0], [0, 2])
    # the dequantised state feeds the next step: s_state * q
    state = np.array([[[10, -20]]], np.int8)
    y, st = oracle.sscan_update(state, np.zeros((1, 1), np.int8), dt, A_log, Bm, np.array([[1, 1]], np.int8), None,
                                None, None, s_x=1.0, s_dt=1.0, s_A=1.0, s_B=1.0, s_C=1.0, s_state=0.5, softplus=False)
    np.testing.assert_allclose(y[0, 0], (5.0 - 10.0) * np.exp(-1.0), rtol=1e-6)
