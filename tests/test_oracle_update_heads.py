"""Pins the CPU oracle's single-step update in the layout with heads (no GPU): it reduces to the one-head
restatement, follows the float64 recurrence written from the mathematics, picks the scale row of the right
(ssd group, head group, dim group, state) and rounds the int8 state half to even."""
import numpy as np
import pytest

import oracle
from oracle import naive
from quamba_amd import synth


def _inputs(B, H, P, N, G, seed, nhg=0, ndg=0):
    g = np.random.default_rng(seed)
    i8 = lambda *shape: g.integers(-127, 128, shape).astype(np.int8)
    d = dict(x=i8(B, H, P), z=i8(B, H, P), dt=i8(B, H, 1), A_log=g.integers(0, 128, (H, 1, 1)).astype(np.int8),
             B=i8(B, G, N), C=i8(B, G, N), D=g.integers(60, 128, (H, 1)).astype(np.int8),
             dt_bias=g.uniform(-4.0, -1.0, (H, 1)).astype(np.float16).astype(np.float32),
             s_dt=np.float32(0.02), s_A=np.float32(np.log(16.0) / 127), s_D=np.float32(1 / 127), s_z=np.float32(0.03))
    if nhg:
        hpg = H // G
        cuts = lambda total, n: np.concatenate([np.sort(g.choice(np.arange(1, total), n - 1, replace=False)), [total]])
        d["head_range"] = np.stack([cuts(hpg, nhg) for _ in range(G)]).astype(np.int32)
        d["dim_range"] = np.stack([np.stack([cuts(P, ndg) for _ in range(nhg)]) for _ in range(G)]).astype(np.int32)
        d["x_scale"] = g.uniform(0.01, 0.05, (G, nhg, ndg)).astype(np.float32)
        d["s_B"] = g.uniform(0.01, 0.03, G).astype(np.float32)
        d["s_C"] = g.uniform(0.01, 0.03, G).astype(np.float32)
        d["state_scale"] = g.uniform(0.002, 0.006, (G, nhg, ndg, N)).astype(np.float32)
    else:
        d["head_range"] = d["dim_range"] = None
        d["x_scale"], d["s_B"], d["s_C"], d["state_scale"] = (np.float32(v) for v in (0.03, 0.02, 0.025, 0.004))
    return d


def _step(d, state, **over):
    kw = dict(x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"], s_D=d["s_D"], s_z=d["s_z"],
              state_scale=d["state_scale"], head_range=d["head_range"], dim_range=d["dim_range"])
    kw.update(over)
    return oracle.ssm_update_heads(state, d["x"], d["dt"], d["A_log"], d["B"], d["C"], d["D"], d["dt_bias"], d["z"], **kw)


def _row_index(d, H, P, G):
    """(G*nhg*ndg index per (head, p)) from a searchsorted formulation of the cumulative end-index tables."""
    hpg = H // G
    idx = np.empty((H, P), int)
    nhg, ndg = d["head_range"].shape[1], d["dim_range"].shape[2]
    for h in range(H):
        g = h // hpg
        hg = int(np.searchsorted(d["head_range"][g], h % hpg, side="right"))
        for p in range(P):
            dg = int(np.searchsorted(d["dim_range"][g, hg], p, side="right"))
            idx[h, p] = (g * nhg + hg) * ndg + dg
    return idx


@pytest.mark.parametrize("fp32_state", [False, True])
def test_one_head_equals_the_mamba1_restatement(fp32_state):
    B, D_, N = 3, 40, 16
    m = synth.mamba1_scan_inputs(B, 1, D_, N, seed=21)
    g = np.random.default_rng(4)
    state = g.standard_normal((B, D_, N)).astype(np.float32) * 0.1 if fp32_state else g.integers(-127, 128, (B, D_, N)).astype(np.int8)
    s_state = np.float32(0.003)
    kw = dict(s_dt=m["s_dt"], s_A=m["s_A"], s_B=m["s_B"], s_C=m["s_C"], s_D=m["s_D"], s_z=m["s_z"])
    y1, st1 = oracle.sscan_update(state, m["u"][:, :, 0], m["dt"][:, :, 0], m["A_log"], m["B"][:, :, 0], m["C"][:, :, 0],
                                  m["D"], m["dt_bias"], m["z"][:, :, 0], s_x=m["s_u"], s_db=m["s_db"], s_state=s_state, **kw)
    bias = np.float32(m["s_db"]) * m["dt_bias"].astype(np.float32)
    y2, st2 = oracle.ssm_update_heads(state[:, None], m["u"][:, None, :, 0], m["dt"][:, None, :, 0], m["A_log"][None],
                                      m["B"][:, None, :, 0], m["C"][:, None, :, 0], m["D"][None], bias[None],
                                      m["z"][:, None, :, 0], x_scale=m["s_u"], state_scale=s_state, **kw)
    np.testing.assert_array_equal(y1, y2[:, 0])
    np.testing.assert_array_equal(st1, st2[:, 0])


def test_uniform_group_scales_equal_the_per_tensor_form():
    B, H, P, N, G = 2, 8, 16, 32, 2
    d = _inputs(B, H, P, N, G, seed=8, nhg=2, ndg=4)
    d["x_scale"][:] = 0.03; d["s_B"][:] = 0.02; d["s_C"][:] = 0.025; d["state_scale"][:] = 0.004
    state = np.random.default_rng(1).standard_normal((B, H, P, N)).astype(np.float32)
    y_g, st_g = _step(d, state)
    y_t, st_t = _step(d, state, x_scale=0.03, s_B=0.02, s_C=0.025, state_scale=0.004, head_range=None, dim_range=None)
    np.testing.assert_array_equal(y_g, y_t)
    np.testing.assert_array_equal(st_g, st_t)


def test_fp32_state_steps_follow_the_float64_recurrence():
    B, H, P, N, G, L = 2, 8, 16, 32, 2, 6
    steps = [_inputs(B, H, P, N, G, seed=100 + t, nhg=2, ndg=4) for t in range(L)]
    d0 = steps[0]
    for s in steps[1:]:                       # parameters stay, inputs change
        for k in ("A_log", "D", "dt_bias", "head_range", "dim_range", "x_scale", "s_B", "s_C", "state_scale"):
            s[k] = d0[k]
    idx = _row_index(d0, H, P, G)
    xs = d0["x_scale"].reshape(-1)[idx].astype(np.float64)                                   # (H, P)
    x = np.stack([s["x"].astype(np.float64) * xs[None] for s in steps], 1)                   # (B, L, H, P)
    dt = np.stack([naive.softplus(s["dt"][..., 0].astype(np.float64) * float(d0["s_dt"]) + d0["dt_bias"][None, :, 0].astype(np.float64))
                   for s in steps], 1)                                                       # (B, L, H)
    A = -np.exp(d0["A_log"][:, 0, 0].astype(np.float64) * float(d0["s_A"]))
    Bm = np.stack([s["B"].astype(np.float64) * d0["s_B"].astype(np.float64)[None, :, None] for s in steps], 1)
    Cm = np.stack([s["C"].astype(np.float64) * d0["s_C"].astype(np.float64)[None, :, None] for s in steps], 1)
    Dv = d0["D"][:, 0].astype(np.float64) * float(d0["s_D"])
    z = np.stack([s["z"].astype(np.float64) * float(d0["s_z"]) for s in steps], 1)
    y64, h64 = naive.ssd_recurrence(x, dt, A, Bm, Cm, Dv, z)
    state = np.zeros((B, H, P, N), np.float32)
    for t, s in enumerate(steps):
        y, state = _step(s, state)
        np.testing.assert_allclose(y, y64[:, t], rtol=2e-5, atol=2e-5 * np.abs(y64).max())
    np.testing.assert_allclose(state, h64, rtol=2e-5, atol=1e-6 * np.abs(h64).max())


def test_int8_state_uses_the_scale_of_its_group_row_and_rounds_half_to_even():
    # zero state, no decay term left (state 0), softplus off, dt = 1: h = B * x exactly; scales are powers of two,
    # different for every (group row, state), so a wrong row or state index changes the quotient
    B, H, P, N, G, nhg, ndg = 1, 8, 8, 4, 2, 2, 2
    d = _inputs(B, H, P, N, G, seed=3, nhg=nhg, ndg=ndg)
    d["dt"] = np.ones((B, H, 1), np.int8); d["dt_bias"] = None
    d["x_scale"][:] = 1.0; d["s_B"][:] = 0.5; d["s_C"][:] = 1.0
    d["x"] = np.random.default_rng(0).integers(-6, 7, (B, H, P)).astype(np.int8)
    d["B"] = np.random.default_rng(1).integers(-7, 8, (B, G, N)).astype(np.int8) | 1        # odd: x*B/2 lands on halves
    rows = G * nhg * ndg
    d["state_scale"] = (2.0 ** -(np.arange(rows * N) % 3)).astype(np.float32).reshape(G, nhg, ndg, N)
    state = np.zeros((B, H, P, N), np.int8)
    _, st = _step(d, state, s_dt=np.float32(1.0), softplus=False)
    idx = _row_index(d, H, P, G)
    hpg = H // G
    want = np.empty((B, H, P, N), np.int64)
    ties = 0
    for h in range(H):
        for p in range(P):
            for n in range(N):
                v = 0.5 * float(d["B"][0, h // hpg, n]) * float(d["x"][0, h, p])
                q = v / float(d["state_scale"].reshape(rows, N)[idx[h, p], n])
                ties += abs(q - np.floor(q) - 0.5) < 1e-9
                want[0, h, p, n] = np.clip(np.rint(q), -128, 127)                           # numpy rint: half to even
    assert ties > 20
    np.testing.assert_array_equal(st, want)


def test_dequantised_state_feeds_the_step_and_y_uses_the_unrounded_state():
    B, H, P, N, G = 1, 2, 4, 4, 1
    d = _inputs(B, H, P, N, G, seed=5, nhg=1, ndg=2)
    d["x"][:] = 0; d["D"] = None; d["z"] = None
    d["dt"] = np.ones((B, H, 1), np.int8); d["dt_bias"] = None
    d["A_log"][:] = 0                                                          # A = -1
    d["C"][:] = 1; d["s_C"][:] = 1.0
    d["state_scale"] = np.array([[[[0.5] * N, [0.25] * N]]], np.float32)
    d["dim_range"] = np.array([[[2, 4]]], np.int32)
    state = np.full((B, H, P, N), 10, np.int8)
    y, st = _step(d, state, s_dt=np.float32(1.0), softplus=False)
    decay = np.exp(-1.0)
    np.testing.assert_allclose(y[0, :, :2], N * 5.0 * decay, rtol=1e-6)
    np.testing.assert_allclose(y[0, :, 2:], N * 2.5 * decay, rtol=1e-6)
    np.testing.assert_array_equal(st, np.full_like(st, int(np.rint(10 * decay))))
