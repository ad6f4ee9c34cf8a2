"""Pins the CPU oracle's SSD chunk-scan restatement (no GPU): float64 step-by-step recurrence,
independence of the chunk size, stage identities and the fp16 rounding helper."""
import ctypes as C

import numpy as np
import pytest

import oracle
from oracle import naive
from quamba_amd import synth


def _run(d, chunk, **kw):
    return oracle.ssd_fwd(d["x"], kw.pop("dt", d["dt"]), d["A_log"], d["B"], d["C"], d["D"], d["z"], d["dt_bias"],
                          chunk_size=chunk, x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                          s_D=d["s_D"], s_z=d["s_z"], head_range=d["head_range"], dim_range=d["dim_range"], **kw)


def _real(d):
    B, L, H, P = d["x"].shape
    G = d["B"].shape[2]
    hpg = H // G
    if d["head_range"] is None:
        xs = np.full((H, P), float(d["x_scale"][0]))
        sB = np.full(G, float(d["s_B"][0])); sC = np.full(G, float(d["s_C"][0]))
    else:
        xs = np.empty((H, P))
        for h in range(H):
            g = h // hpg
            hg = int(np.sum((h % hpg) >= d["head_range"][g]))
            for p in range(P):
                dg = int(np.sum(p >= d["dim_range"][g, hg]))
                xs[h, p] = d["x_scale"][g, hg, dg]
        sB, sC = d["s_B"].astype(np.float64), d["s_C"].astype(np.float64)
    x = d["x"].astype(np.float64) * xs[None, None]
    dt = synth.softplus(d["dt"].astype(np.float64) * float(d["s_dt"]) + d["dt_bias"].astype(np.float64)[None, None])
    A = -np.exp(d["A_log"].astype(np.float64) * float(d["s_A"]))
    Bm = d["B"].astype(np.float64) * sB[None, None, :, None]
    Cm = d["C"].astype(np.float64) * sC[None, None, :, None]
    D = d["D"].astype(np.float64) * float(d["s_D"])
    z = None if d["z"] is None else d["z"].astype(np.float64) * float(d["s_z"])
    return x, dt, A, Bm, Cm, D, z


def test_f16_rounding_helper_matches_numpy():
    l = oracle.lib()
    l.qo_f16_round.restype = C.c_float
    l.qo_f16_round.argtypes = [C.c_float]
    g = np.random.default_rng(0)
    vals = np.concatenate([g.standard_normal(2000) * 10.0 ** g.integers(-8, 5, 2000), [0.0, 65504.0, 65519.0, 65520.0, 1e-8,
                           5.96e-8, 2049.0, 2051.0, -2049.0]]).astype(np.float32)
    for v in vals:
        assert l.qo_f16_round(C.c_float(float(v))) == np.float32(np.float16(v)), v


@pytest.mark.parametrize("grouped,with_z", [(False, False), (True, True)])
def test_against_float64_recurrence(grouped, with_z):
    d = synth.mamba2_ssd_inputs(2, 70, 8, 8, 16, 2, seed=3, grouped=grouped, nhead_groups=2, ndim_groups=2, with_z=with_z)
    r = _run(d, chunk=32)
    x, dt, A, Bm, Cm, D, z = _real(d)
    y64, h64 = naive.ssd_recurrence(x, dt, A, Bm, Cm, D, z)
    # fp16 operand rounding (2^-11 relative per factor) bounds the agreement
    assert np.abs(r["y"] - y64).max() <= 4e-3 * np.abs(y64).max()
    assert np.sum((r["y"] - y64) ** 2) / np.sum(y64 ** 2) < 1e-6
    assert np.abs(r["final_f32"] - h64).max() <= 2e-3 * np.abs(h64).max()


def test_result_does_not_depend_on_the_chunk_size():
    d = synth.mamba2_ssd_inputs(1, 96, 4, 8, 16, 1, seed=5)
    a, b, c = _run(d, chunk=32), _run(d, chunk=96), _run(d, chunk=64)
    for other in (b, c):
        np.testing.assert_allclose(other["y"], a["y"], rtol=0, atol=4e-3 * np.abs(a["y"]).max())
        np.testing.assert_allclose(other["final_f32"], a["final_f32"], rtol=0, atol=2e-3 * np.abs(a["final_f32"]).max())


def test_stage_identities():
    d = synth.mamba2_ssd_inputs(1, 64, 4, 8, 16, 2, seed=7)
    r = _run(d, chunk=32, stages=True)
    x, dt, A, Bm, Cm, D, z = _real(d)
    # stage 1: dt and the within-chunk cumulative sum of dt*A
    dt_c = dt.transpose(0, 2, 1).reshape(1, 4, 2, 32)
    np.testing.assert_allclose(r["dt"], dt_c, rtol=1e-5)
    np.testing.assert_allclose(r["dA_cumsum"], np.cumsum(dt_c * A[None, :, None, None], axis=-1), rtol=1e-5)
    # stage 4: CB is an exact integer matrix product times the two scales
    Ci = d["C"].astype(np.int64).reshape(1, 2, 32, 2, 16)
    Bi = d["B"].astype(np.int64).reshape(1, 2, 32, 2, 16)
    cb = np.einsum("bcmgn,bckgn->bcgmk", Ci, Bi) * float(d["s_C"][0]) * float(d["s_B"][0])
    np.testing.assert_allclose(r["CB"], cb, rtol=1e-6)
    # stage 2: the state of chunk c equals the recurrence restricted to the chunk from a zero state
    for c in range(2):
        sl = slice(32 * c, 32 * c + 32)
        _, h = naive.ssd_recurrence(x[:, sl], dt[:, sl], A, Bm[:, sl], Cm[:, sl])
        assert np.abs(r["chunk_states"][:, c] - h).max() <= 2e-3 * np.abs(h).max()
    # stage 3: the state entering chunk 1 is the state after chunk 0, held in fp16
    np.testing.assert_array_equal(r["prev_states"][:, 0], 0)
    np.testing.assert_array_equal(r["prev_states"][:, 1], r["chunk_states"][:, 0].astype(np.float16).astype(np.float32))


def test_fp32_dt_entry_point_and_ragged_tail_and_final_quant():
    d = synth.mamba2_ssd_inputs(1, 45, 4, 8, 16, 1, seed=9)          # 45 = 32 + 13: ragged last chunk
    a = _run(d, chunk=32)
    dt_proc = synth.softplus(d["dt"].astype(np.float32) * d["s_dt"] + d["dt_bias"].astype(np.float32)[None, None]).astype(np.float32)
    b = _run(d, chunk=32, dt=dt_proc)
    np.testing.assert_allclose(b["y"], a["y"], rtol=1e-3, atol=1e-4)
    s = float(np.abs(a["final_f32"]).max() / 127)
    c = _run(d, chunk=32, state_scale=s)
    want = np.clip(np.rint(a["final_f32"].astype(np.float16).astype(np.float32) / np.float32(s)), -128, 127)
    diff = np.abs(c["final_i8"].astype(int) - want.astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.01
    assert np.abs(c["final_i8"]).max() == 127
