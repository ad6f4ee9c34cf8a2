"""End-to-end parity of the assembled Mamba2 mixer (W4A8QMamba2) against the same chain of CPU oracle
functions: in_proj and conv outputs bit-exact, the fp16 stages and the final projection within the SSD
scan's tolerance."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import W4A8QMamba2
from quamba_amd import w4a8_utils as wu

pytestmark = pytest.mark.gpu

D_MODEL, D_STATE, HEADDIM, NGROUPS, CHUNK = 256, 64, 64, 2, 64


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _w4(g, n, k):
    """Random grouped 4-bit layer: codes (n, k), fp16 group scales (k/128, n), fp32 channel scales (n)."""
    codes = g.integers(0, 16, (n, k)).astype(np.uint8)
    sg = g.uniform(2.0, 15.8, (k // 128, n)).astype(np.float16)
    return codes, sg


def _mixer(dev, seed=0):
    g = np.random.default_rng(seed)
    m = W4A8QMamba2(D_MODEL, D_STATE, 4, 2, HEADDIM, ngroups=NGROUPS, chunk_size=CHUNK, device=dev, state_dtype=torch.float32,
                    x_nhead_group=2, x_ndim_group=2)
    D, H, G, N = m.d_inner, m.nheads, NGROUPS, D_STATE
    w = {}
    # in_proj: per-segment output scales folded into the channel scale, as W4A8B8O8LinearParallel.from_fp16 does
    n_in = m.in_proj.size_n
    codes, sg = _w4(g, n_in, D_MODEL)
    s_ch = (g.uniform(0.5, 1.5, n_in) * 0.5 / np.sqrt(D_MODEL) / 8 / 4.6).astype(np.float32)
    w["in"] = (codes, sg, s_ch, np.float32(0.9))
    m.in_proj.weight = wu.pack_w4a8(torch.from_numpy(codes.T.astype(np.int32))).to(dev)
    m.in_proj.s_group, m.in_proj.s_channel = _t(sg, dev), _t(s_ch[None], dev)
    m.in_proj.input_scale = torch.tensor(0.9, device=dev)
    # conv over [x | B | C]
    dim = D + 2 * G * N
    w["conv_w"], w["conv_b"] = g.integers(-127, 128, (dim, 4)).astype(np.int8), g.integers(-127, 128, dim).astype(np.int8)
    cs = dict(scales_in=[0.03, 0.025, 0.028], scales_w=[0.004, 0.0045, 0.0038], scales_b=[0.002, 0.0021, 0.0019],
              x_out_scales=(0.01 + 0.004 * g.random((G, 2, 2))).astype(np.float32),
              B_out_scales=np.array([0.011, 0.012], np.float32), C_out_scales=np.array([0.0115, 0.0105], np.float32),
              x_head_group_range=np.array([[1, 4], [3, 4]], np.int32),           # 4 heads per ssd group
              x_dim_group_range=np.array([[[16, 64], [40, 64]], [[8, 64], [32, 64]]], np.int32))
    w["conv"] = cs
    c = m.conv1d
    c.weight, c.bias = _t(w["conv_w"], dev), _t(w["conv_b"], dev)
    c.x_scale, c.B_scale, c.C_scale = cs["scales_in"]
    c.wx_scale, c.wB_scale, c.wC_scale = cs["scales_w"]
    c.bx_scale, c.bB_scale, c.bC_scale = cs["scales_b"]
    c.x_out_scales, c.B_out_scales, c.C_out_scales = _t(cs["x_out_scales"], dev), _t(cs["B_out_scales"], dev), _t(cs["C_out_scales"], dev)
    c.x_head_group_range, c.x_dim_group_range = _t(cs["x_head_group_range"], dev), _t(cs["x_dim_group_range"], dev)
    # SSD scan: its input scales are the conv's output scales
    q = m.qchunk_scan
    w["A_log"] = g.integers(0, 100, H).astype(np.int8)
    w["Dq"] = g.integers(-127, 128, H).astype(np.int8)
    w["dt_bias"] = (g.uniform(-4, -2, H)).astype(np.float16)
    w["ssd"] = dict(s_dt=0.03, s_A=0.028, s_D=0.008)
    q.A_log, q.D, q.dt_bias = _t(w["A_log"], dev), _t(w["Dq"], dev), _t(w["dt_bias"], dev)
    q.A_log_scale = torch.tensor(0.028, device=dev)
    q.D_scale = torch.tensor(0.008, device=dev)
    q.dt_scale = torch.tensor(0.03, device=dev)
    q.x_scales, q.B_scale, q.C_scale = c.x_out_scales, c.B_out_scales, c.C_out_scales
    q.x_head_group_range, q.x_dim_group_range = c.x_head_group_range, c.x_dim_group_range
    q.ssm_state_scale = torch.full((G, 2, 2, N), 0.05, device=dev)
    # norm, Hadamard, out_proj
    w["norm_w"] = (1 + 0.2 * g.standard_normal(D)).astype(np.float16)
    m.norm.weight = _t(w["norm_w"], dev)
    m.norm.z_scale = 0.03
    m.had.x_H_scale = 0.04
    codes, sg = _w4(g, m.out_proj.size_n, D)
    s_ch = (g.uniform(0.5, 1.5, m.out_proj.size_n) * 1e-4).astype(np.float32)
    w["out"] = (codes, sg, s_ch, np.float32(0.04))
    m.out_proj.weight = wu.pack_w4a8(torch.from_numpy(codes.T.astype(np.int32))).to(dev)
    m.out_proj.s_group, m.out_proj.s_channel = _t(sg, dev), _t(s_ch[None], dev)
    m.out_proj.input_scale = torch.tensor(0.04, device=dev)
    return m, w


def _oracle_forward(m, w, u):
    Bsz, L, _ = u.shape
    D, H, G, N, P = m.d_inner, m.nheads, NGROUPS, D_STATE, HEADDIM
    codes, sg, s_ch, s_in = w["in"]
    zxbcdt = oracle.gemm_w4a8(u.reshape(Bsz * L, -1), codes, sg, s_ch, [s_in])[3][:, :2 * D + 2 * G * N + H]
    z, xBC, dt = zxbcdt[:, :D], zxbcdt[:, D:2 * D + 2 * G * N], zxbcdt[:, 2 * D + 2 * G * N:]
    cs = w["conv"]
    chan = oracle.quamba2_conv_channel_scales(D, P, N, G, cs["scales_in"], cs["scales_w"], cs["scales_b"], cs["x_out_scales"],
                                              cs["B_out_scales"], cs["C_out_scales"], cs["x_head_group_range"], cs["x_dim_group_range"])
    xBC_t = np.ascontiguousarray(xBC.reshape(Bsz, L, -1).transpose(0, 2, 1))
    x, Bm, Cm = oracle.quamba2_conv1d_fwd(xBC_t, w["conv_w"], w["conv_b"], *chan, D, G * N)
    to_blhp = lambda a, h, p: np.ascontiguousarray(a.transpose(0, 2, 1)).reshape(Bsz, L, h, p)
    ssd = oracle.ssd_fwd(to_blhp(x, H, P), np.ascontiguousarray(dt.reshape(Bsz, L, H)), w["A_log"], to_blhp(Bm, G, N),
                         to_blhp(Cm, G, N), D=w["Dq"], dt_bias=w["dt_bias"], chunk_size=CHUNK, x_scale=cs["x_out_scales"],
                         s_dt=w["ssd"]["s_dt"], s_A=w["ssd"]["s_A"], s_B=cs["B_out_scales"], s_C=cs["C_out_scales"],
                         s_D=w["ssd"]["s_D"], head_range=cs["x_head_group_range"], dim_range=cs["x_dim_group_range"])
    y16 = ssd["y"].astype(np.float16).reshape(Bsz * L, D)
    _, yn, _ = oracle.rmsnorm_gated(y16, w["norm_w"], np.ascontiguousarray(z), eps=1e-5, z_scale=0.03, group_size=D // G,
                                    norm_before_gate=False)
    yq = oracle.hadamard_quant(yn, np.float32(1.0 / np.sqrt(D) / 0.04))
    codes, sg, s_ch, s_in = w["out"]
    out = oracle.gemm_w4a8(yq, codes, sg, s_ch, [s_in])[2][:, :D_MODEL].astype(np.float16)
    return dict(zxbcdt=zxbcdt, x=x, B=Bm, C=Cm, y=ssd["y"], state=ssd["final_f32"], yn=yn, yq=yq, out=out.reshape(Bsz, L, -1),
                xBC_t=xBC_t)


def test_forward_matches_the_oracle_chain(dev):
    m, w = _mixer(dev)
    g = np.random.default_rng(1)
    u = g.integers(-127, 128, (2, 150, D_MODEL)).astype(np.int8)           # 150 = two chunks of 64 and a ragged one
    want = _oracle_forward(m, w, u)
    conv_state, ssm_state = m.allocate_inference_cache(2)
    got = m(_t(u, dev), conv_state=conv_state, ssm_state=ssm_state)
    assert got.shape == (2, 150, D_MODEL) and got.dtype == torch.float16
    for k in ("x", "B", "C", "yq"):
        assert np.abs(want[k]).max() > 40, k
    # int8 stages: bit-exact
    d = m.in_proj(_t(u, dev)).reshape(300, -1).cpu().numpy()
    np.testing.assert_array_equal(d, want["zxbcdt"])
    xs, Bs, Cs = m.conv1d(m._split(m.in_proj(_t(u, dev)))[1].transpose(1, 2))
    np.testing.assert_array_equal(xs.cpu().numpy(), want["x"])
    np.testing.assert_array_equal(Cs.cpu().numpy(), want["C"])
    # fp16 stages and the projection
    out = got.float().cpu().numpy()
    ref = want["out"].astype(np.float32)
    scale = np.abs(ref).max()
    assert scale > 0.05
    assert np.max(np.abs(out - ref)) <= 0.06 * scale and np.mean(np.abs(out - ref)) <= 0.01 * scale
    np.testing.assert_allclose(ssm_state.cpu().numpy(), want["state"], rtol=2e-3, atol=2e-3 * np.abs(want["state"]).max())
    np.testing.assert_array_equal(conv_state.cpu().numpy(), want["xBC_t"][:, :, -4:])


def test_step_runs_on_the_cached_states(dev):
    m, w = _mixer(dev, seed=2)
    g = np.random.default_rng(3)
    u = g.integers(-127, 128, (2, 70, D_MODEL)).astype(np.int8)
    conv_state, ssm_state = m.allocate_inference_cache(2)
    full = m(_t(u, dev), conv_state=conv_state, ssm_state=ssm_state)
    # one more token through step == the last position of a forward over the extended sequence
    nxt = g.integers(-127, 128, (2, 1, D_MODEL)).astype(np.int8)
    out_step, _, _ = m.step(_t(nxt, dev), conv_state, ssm_state)
    ref = m(_t(np.concatenate([u, nxt], axis=1), dev))[:, -1:]
    assert out_step.shape == (2, 1, D_MODEL)
    scale = ref.float().abs().max().item()
    assert (out_step.float() - ref.float()).abs().max().item() <= 0.08 * scale + 1e-3
    assert full.shape == (2, 70, D_MODEL)
