"""GPU parity of the Mamba2 SSD chunk scan and its single-step update against the CPU oracle.
fp16 outputs: rtol 1e-2 / atol 1e-2 (relative to the output scale); fp32 states 1e-3 relative."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import Quamba2ChunkScan, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _oracle(d, chunk, **kw):
    return oracle.ssd_fwd(d["x"], kw.pop("dt", d["dt"]), d["A_log"], d["B"], d["C"], d["D"], d["z"], d["dt_bias"],
                          chunk_size=chunk, x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                          s_D=d["s_D"], s_z=d["s_z"], head_range=d["head_range"], dim_range=d["dim_range"], **kw)


def _gpu(d, dev, chunk, state_scale=None, dt=None, final_dtype=torch.float32, **kw):
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    return ops.ssd_chunk_scan_combined_fwd(
        _t(d["x"], dev), s(d["x_scale"]), _t(d["dt"] if dt is None else dt, dev), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
        _t(d["B"], dev), s(d["s_B"]), _t(d["C"], dev), s(d["s_C"]), None if state_scale is None else s(state_scale), chunk,
        q_D=_t(d["D"], dev), D_scale=s(d["s_D"]), q_z=_t(d["z"], dev), z_scale=s(d["s_z"]), dt_bias=_t(d["dt_bias"], dev),
        dt_softplus=True, x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev),
        final_state_dtype=final_dtype, **kw)


def _check_y(y_gpu, y_ref):
    got = y_gpu.float().cpu().numpy()
    scale = np.abs(y_ref).max()
    np.testing.assert_allclose(got / scale, y_ref.astype(np.float16).astype(np.float32) / scale, rtol=1e-2, atol=1e-2)
    assert np.sum((got - y_ref) ** 2) / np.sum(y_ref ** 2) < 1e-4


# batch, seqlen, nheads, dstate, ngroups, chunk
SHAPES = [(1, 64, 2, 128, 1, 64), (2, 33, 4, 128, 1, 64), (1, 89, 4, 64, 2, 64), (2, 300, 8, 64, 2, 128),
          (1, 512, 8, 128, 1, 256), (1, 1024, 4, 128, 1, 256), (1, 130, 4, 128, 4, 128),
          # fewer states than the kernels are built for (the 16-state row of test_ssd_combined.py:25, and 32, 96)
          (1, 33, 24, 16, 1, 128), (2, 200, 4, 32, 2, 64), (1, 150, 4, 96, 1, 128)]


@pytest.mark.parametrize("B,L,H,N,G,Q", SHAPES)
def test_forward_matches_oracle(dev, B, L, H, N, G, Q):
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=L + H)
    ref = _oracle(d, Q)
    y, final = _gpu(d, dev, Q)
    assert y.shape == (B, L, H, 64) and y.dtype == torch.float16 and final.shape == (B, H, 64, N)
    _check_y(y, ref["y"])
    got = final.cpu().numpy()
    assert np.abs(got - ref["final_f32"]).max() <= 1e-3 * np.abs(ref["final_f32"]).max()


def test_every_stage_matches_the_oracle(dev):
    B, L, H, N, G, Q = 2, 200, 4, 128, 2, 64
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=77)
    ref = _oracle(d, Q, stages=True)
    y, final, ws = _gpu(d, dev, Q, return_workspace=True)
    nc = (L + Q - 1) // Q
    a256 = lambda v: (v + 255) & ~255
    off, parts = 0, {}
    for name, shape, dt in [("dt", (B, H, nc, Q), torch.float32), ("dA_cumsum", (B, H, nc, Q), torch.float32),
                            ("CB", (B, nc, G, Q, Q), torch.float16), ("prev_states", (B, nc, H, 64, N), torch.float16)]:
        n = int(np.prod(shape)) * (4 if dt == torch.float32 else 2)
        parts[name] = ws[off:off + n].view(dt).view(shape).float().cpu().numpy()
        off = a256(off + n)
    np.testing.assert_allclose(parts["dt"], ref["dt"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(parts["dA_cumsum"], ref["dA_cumsum"], rtol=1e-5, atol=1e-8)
    # C B^T is kept in fp16, divided by 16; Q == 64: one tile, all of it written
    np.testing.assert_allclose(parts["CB"] * 16.0, ref["CB"], rtol=1e-3, atol=1e-3 * np.abs(ref["CB"]).max())
    # the fp32 chunk states stay in registers; the states entering each chunk (their running sum) are checked
    assert np.abs(parts["prev_states"] - ref["prev_states"]).max() <= 1e-3 * np.abs(ref["prev_states"]).max()


@pytest.mark.parametrize("with_z,d_has_hdim", [(True, False), (False, True)])
def test_grouped_scales_z_gate_and_int8_state(dev, with_z, d_has_hdim):
    B, L, H, N, G, Q = 2, 150, 16, 128, 2, 128
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=5, grouped=True, nhead_groups=4, ndim_groups=4, with_z=with_z)
    if d_has_hdim:
        d["D"] = np.random.default_rng(1).integers(60, 128, (H, 64)).astype(np.int8)
    ref = _oracle(d, Q)
    g = np.random.default_rng(2)
    state_scale = (np.abs(ref["final_f32"]).max() / 127 * g.uniform(0.8, 1.2, (G, 4, 4, N))).astype(np.float32)
    ref = _oracle(d, Q, state_scale=state_scale)
    y, final = _gpu(d, dev, Q, state_scale=state_scale, final_dtype=torch.int8)
    _check_y(y, ref["y"])
    assert final.dtype == torch.int8
    diff = np.abs(final.cpu().numpy().astype(int) - ref["final_i8"].astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02
    assert np.abs(ref["final_i8"]).max() > 100


def test_fp32_step_sizes_entry_point(dev):
    d = synth.mamba2_ssd_inputs(1, 256, 4, 64, 128, 1, seed=9)
    dt_proc = synth.softplus(d["dt"].astype(np.float32) * d["s_dt"] + d["dt_bias"].astype(np.float32)[None, None]).astype(np.float32)
    ref = _oracle(d, 128, dt=dt_proc)
    y, final = _gpu(d, dev, 128, dt=dt_proc)
    _check_y(y, ref["y"])


def test_module_forward_then_update_continue_the_sequence(dev):
    B, L, H, N, G, Q = 2, 128, 8, 128, 2, 64
    d = synth.mamba2_ssd_inputs(B, L + 3, H, 64, N, G, seed=13, grouped=True, nhead_groups=2, ndim_groups=2)
    ref = _oracle(d, 131)                     # one chunk covering everything: the recurrence itself
    ref = _oracle(d, Q)
    A_log = torch.from_numpy(d["A_log"].astype(np.float32) * d["s_A"]).to(dev)
    q = Quamba2ChunkScan.from_fp16(
        H * 64, 64, N, G, torch.from_numpy(d["x_scale"]), _t(d["head_range"], dev), _t(d["dim_range"], dev), A_log, Q,
        ssm_state_scale=torch.ones(G, 2, 2, N), D=torch.ones(H, device=dev), dt_bias=_t(d["dt_bias"], dev),
        dt_scale=torch.tensor(float(d["s_dt"])), B_scale=torch.from_numpy(d["s_B"]), C_scale=torch.from_numpy(d["s_C"]))
    np.testing.assert_array_equal(q.A_log.cpu().numpy(), d["A_log"])
    assert q.dt_bias.dtype == torch.float16 and q.x_scales.shape == (G, 2, 2) and q.ssm_state_scale.shape == (G, 2, 2, N)
    cut = lambda a: _t(a[:, :L], dev)
    y, state = q(cut(d["x"]), cut(d["dt"]), cut(d["B"]), cut(d["C"]), return_final_states=True, state_dtype=torch.float32)
    _check_y(y, ref["y"][:, :L])
    for t in range(L, L + 3):
        yt = q.update(state, _t(d["x"][:, t].reshape(B, -1), dev), _t(d["dt"][:, t], dev), _t(d["B"][:, t].reshape(B, -1), dev),
                      _t(d["C"][:, t].reshape(B, -1), dev))
        want = ref["y"][:, t]
        np.testing.assert_allclose(yt.float().cpu().numpy() / np.abs(want).max(), want / np.abs(want).max(), rtol=1e-2, atol=1e-2)
    assert np.abs(state.cpu().numpy() - ref["final_f32"]).max() <= 2e-3 * np.abs(ref["final_f32"]).max()


def test_errors(dev):
    d = synth.mamba2_ssd_inputs(1, 64, 2, 64, 128, 1, seed=1)
    with pytest.raises(NotImplementedError):
        _gpu(d, dev, 48)                                  # chunk sizes other than 64 / 128 / 256
    with pytest.raises(NotImplementedError, match="seq_idx"):
        _gpu(d, dev, 64, seq_idx=torch.zeros(1, 64, device=dev))
    d2 = synth.mamba2_ssd_inputs(1, 64, 2, 32, 128, 1, seed=1)
    with pytest.raises(NotImplementedError):
        _gpu(d2, dev, 64)                                 # head dimensions other than 64
