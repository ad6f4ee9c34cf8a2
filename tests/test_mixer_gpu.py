"""End-to-end parity of the assembled Mamba1 mixer (W8A8QMamba) against the same chain of CPU oracle
functions: every int8 tensor up to the scan bit-exact, the fp16 scan output and the final projection
within the scan's tolerance; the one-token step against the oracle's update chain."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import W8A8QMamba

pytestmark = pytest.mark.gpu

D_MODEL, D_STATE, D_CONV = 256, 16, 4


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _mixer(dev, seed=0, state_dtype=torch.float32):
    g = np.random.default_rng(seed)
    m = W8A8QMamba(D_MODEL, D_STATE, D_CONV, device=dev, state_dtype=state_dtype)
    D, R, N = m.d_inner, m.dt_rank, D_STATE
    ri = lambda *s: g.integers(-127, 128, s).astype(np.int8)
    w = dict(in_proj=ri(2 * D, D_MODEL), x_proj=ri(R + 2 * N, D), dt_proj=ri(D, R), out_proj=ri(D_MODEL, D),
             conv_w=ri(D, D_CONV), conv_b=ri(D), A_log=g.integers(0, 100, (D, N)).astype(np.int8), Dq=ri(D), dt_bias=ri(D))
    # (a = input/output scale ratio, b = weight scale) of each int8 linear, chosen so outputs use the int8 range
    s = dict(in_a=0.9, in_b=2.4e-3 / np.sqrt(D_MODEL) * 16, x_a=1.1, x_b=2.0e-3 / np.sqrt(D) * 16, dt_a=0.8, dt_b=0.5e-2,
             out_a=0.02, out_b=0.003, conv_x=0.03, conv_w=0.004, conv_b=0.002, conv_o=0.012,
             u=0.012, dt=0.03, A=0.028, B=0.02, C=0.02, z=0.03, Dsc=0.008, db=0.02, state=0.05, had=0.05)
    for name, a, b in (("in_proj", s["in_a"], s["in_b"]), ("x_proj", s["x_a"], s["x_b"]), ("dt_proj", s["dt_a"], s["dt_b"]),
                       ("out_proj", s["out_a"], s["out_b"])):
        lin = getattr(m, name)
        lin._set_weight(_t(w[name], dev))
        lin.a = torch.tensor([[a]], dtype=torch.float32, device=dev)
        lin.b = torch.tensor([[b]], dtype=torch.float32, device=dev)
        lin.alpha = float(np.float32(a) * np.float32(b))
    m.conv1d.weight, m.conv1d.bias = _t(w["conv_w"], dev), _t(w["conv_b"], dev)
    m.conv1d.input_scale, m.conv1d.weight_scale, m.conv1d.bias_scale, m.conv1d.output_scale = (
        s["conv_x"], s["conv_w"], s["conv_b"], s["conv_o"])
    sc = m.selective_scan
    sc.A_log, sc.D, sc.dt_bias = _t(w["A_log"], dev), _t(w["Dq"], dev), _t(w["dt_bias"], dev)
    for name, key in (("A_scale", "A"), ("D_scale", "Dsc"), ("dt_bias_scale", "db"), ("u_scale", "u"), ("dt_scale", "dt"),
                      ("B_scale", "B"), ("C_scale", "C"), ("z_scale", "z"), ("ssm_state_scale", "state")):
        setattr(sc, name, torch.tensor(s[key], dtype=torch.float32, device=dev))
    m.had.x_H_scale = s["had"]
    return m, w, s


def _oracle_forward(m, w, s, hidden):
    """The chain of quamba/qMambaLayer.py:911-943 on the CPU oracle.  hidden int8 (B, L, d_model)."""
    B, L, _ = hidden.shape
    D, R, N = m.d_inner, m.dt_rank, D_STATE
    h2 = hidden.reshape(B * L, -1)
    # to_seqlen_last computes W x^T: the weight scale is the row scale, the activation scale the column scale
    xz = oracle.gemm_w8a8(w["in_proj"], h2, [s["in_b"]], [s["in_a"]])[2].reshape(2 * D, B, L).transpose(1, 0, 2)
    x_in, z = np.ascontiguousarray(xz[:, :D]), np.ascontiguousarray(xz[:, D:])
    x = oracle.conv1d_fwd(x_in, w["conv_w"], w["conv_b"], s["conv_x"], s["conv_w"], s["conv_b"], s["conv_o"])
    x_dbl = oracle.gemm_w8a8(np.ascontiguousarray(x.transpose(0, 2, 1)).reshape(B * L, D), w["x_proj"], [s["x_a"]], [s["x_b"]])[2]
    dt_in, Bm, Cm = x_dbl[:, :R], x_dbl[:, R:R + N], x_dbl[:, R + N:]
    dt = oracle.gemm_w8a8(w["dt_proj"], np.ascontiguousarray(dt_in), [s["dt_b"]], [s["dt_a"]])[2].reshape(D, B, L).transpose(1, 0, 2)
    Bm = np.ascontiguousarray(Bm.reshape(B, L, N).transpose(0, 2, 1))
    Cm = np.ascontiguousarray(Cm.reshape(B, L, N).transpose(0, 2, 1))
    y, _, state = oracle.sscan_fwd(x, np.ascontiguousarray(dt), w["A_log"], Bm, Cm, w["Dq"], w["dt_bias"], z, s_u=s["u"],
                                   s_delta=s["dt"], s_A=s["A"], s_B=s["B"], s_C=s["C"], s_D=s["Dsc"], s_db=s["db"], s_z=s["z"])
    y16 = y.astype(np.float16)
    yq = oracle.hadamard_quant(y16, np.float32(1.0 / np.sqrt(D) / s["had"]))
    out = oracle.gemm_w8a8(yq.reshape(B * L, D), w["out_proj"], [s["out_a"]], [s["out_b"]])[1].astype(np.float16)
    return dict(x_in=x_in, z=z, x=x, dt=np.ascontiguousarray(dt), B=Bm, C=Cm, y=y, state=state, yq=yq,
                out=out.reshape(B, L, -1))


def test_forward_matches_the_oracle_chain(dev):
    m, w, s = _mixer(dev)
    g = np.random.default_rng(1)
    hidden = g.integers(-127, 128, (2, 48, D_MODEL)).astype(np.int8)
    want = _oracle_forward(m, w, s, hidden)
    conv_state, ssm_state = m.allocate_inference_cache(2)
    got = m(_t(hidden, dev), conv_state=conv_state, ssm_state=ssm_state)
    assert got.shape == (2, 48, D_MODEL) and got.dtype == torch.float16
    # every stage exercised: the intermediate tensors are not degenerate
    for k in ("x", "dt", "B", "yq"):
        assert np.abs(want[k]).max() > 40, k
    out = got.float().cpu().numpy()
    ref = want["out"].astype(np.float32)
    # the scan output is fp16 with tolerance, so a few Hadamard outputs may sit one step off; the final
    # projection averages over d_inner such steps
    step = s["out_a"] * s["out_b"] * 127 * np.sqrt(m.d_inner)
    assert np.max(np.abs(out - ref)) <= 4 * step + 2e-2 * np.abs(ref).max()
    assert np.mean(np.abs(out - ref)) <= 0.25 * step
    np.testing.assert_allclose(ssm_state.cpu().numpy(), want["state"], rtol=1e-3, atol=1e-3 * np.abs(want["state"]).max())
    np.testing.assert_array_equal(conv_state.cpu().numpy(), want["x_in"][:, :, -D_CONV:])


def test_int8_stages_are_bit_exact(dev):
    m, w, s = _mixer(dev, seed=3)
    g = np.random.default_rng(2)
    hidden = g.integers(-127, 128, (1, 33, D_MODEL)).astype(np.int8)
    want = _oracle_forward(m, w, s, hidden)
    h = _t(hidden, dev)
    xz = m.in_proj.to_seqlen_last(h)
    x_in, z = xz.chunk(2, dim=1)
    np.testing.assert_array_equal(x_in.cpu().numpy(), want["x_in"])
    np.testing.assert_array_equal(z.cpu().numpy(), want["z"])
    x = m.conv1d(x_in)
    np.testing.assert_array_equal(x.cpu().numpy(), want["x"])
    x_dbl = m.x_proj(x.transpose(1, 2).contiguous())
    dt = m.dt_proj.to_seqlen_last(x_dbl[..., :m.dt_rank].contiguous())
    np.testing.assert_array_equal(dt.cpu().numpy(), want["dt"])
    np.testing.assert_array_equal(x_dbl[..., m.dt_rank:m.dt_rank + D_STATE].transpose(1, 2).cpu().numpy(), want["B"])


def test_step_matches_the_oracle_update_chain(dev):
    m, w, s = _mixer(dev, seed=5)
    g = np.random.default_rng(4)
    B = 3
    D, R, N = m.d_inner, m.dt_rank, D_STATE
    conv_state = g.integers(-127, 128, (B, D, D_CONV)).astype(np.int8)
    ssm_state = (g.standard_normal((B, D, N)) * 0.1).astype(np.float32)
    d_conv, d_ssm = _t(conv_state, dev), _t(ssm_state, dev)
    for _ in range(3):
        hidden = g.integers(-127, 128, (B, 1, D_MODEL)).astype(np.int8)
        xz = oracle.gemm_w8a8(hidden[:, 0], w["in_proj"], [s["in_a"]], [s["in_b"]])[2]
        x, conv_state = oracle.conv1d_update(np.ascontiguousarray(xz[:, :D]), conv_state, w["conv_w"], w["conv_b"],
                                             s["conv_x"], s["conv_w"], s["conv_b"], s["conv_o"])
        x_db = oracle.gemm_w8a8(x, w["x_proj"], [s["x_a"]], [s["x_b"]])[2]
        dt = oracle.gemm_w8a8(np.ascontiguousarray(x_db[:, :R]), w["dt_proj"], [s["dt_a"]], [s["dt_b"]])[2]
        y, ssm_state = oracle.sscan_update(ssm_state, x, dt, w["A_log"], np.ascontiguousarray(x_db[:, R:R + N]),
                                           np.ascontiguousarray(x_db[:, R + N:]), w["Dq"], w["dt_bias"],
                                           np.ascontiguousarray(xz[:, D:]), s_x=s["u"], s_dt=s["dt"], s_A=s["A"], s_B=s["B"],
                                           s_C=s["C"], s_D=s["Dsc"], s_db=s["db"], s_z=s["z"])
        yq = oracle.hadamard_quant(y.astype(np.float16), np.float32(1.0 / np.sqrt(D) / s["had"]))
        want = oracle.gemm_w8a8(yq, w["out_proj"], [s["out_a"]], [s["out_b"]])[1].astype(np.float16)
        got, _, _ = m.step(_t(hidden, dev), d_conv, d_ssm)
        np.testing.assert_array_equal(d_conv.cpu().numpy(), conv_state)
        np.testing.assert_allclose(d_ssm.cpu().numpy(), ssm_state, rtol=1e-3, atol=1e-4)
        step = s["out_a"] * s["out_b"] * 127 * np.sqrt(D)
        assert np.max(np.abs(got[:, 0].float().cpu().numpy() - want.astype(np.float32))) <= 4 * step + 1e-2


def test_inference_cache_path(dev):
    m, _, _ = _mixer(dev, seed=7)
    m.layer_idx = 0

    class Params:
        seqlen_offset = 0
        key_value_memory_dict = {}

    p = Params()
    h = torch.randint(-127, 128, (2, 16, D_MODEL), dtype=torch.int8, device=dev)
    out = m(h, inference_params=p)
    assert out.shape == (2, 16, D_MODEL) and 0 in p.key_value_memory_dict
    p.seqlen_offset = 16
    out1 = m(h[:, :1], inference_params=p)
    assert out1.shape == (2, 1, D_MODEL) and torch.isfinite(out1.float()).all()
