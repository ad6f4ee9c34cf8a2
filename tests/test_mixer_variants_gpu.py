"""The other two precisions of the mixers (W4A8QMamba, W8A8QMamba2): the chains are the ones tested end to end
against the oracle in test_mixer_gpu.py / test_mixer2_gpu.py with the linear classes exchanged, so the check
here is the one that involves every kernel of the class twice: one more token through ``step`` (few-rows GEMMs,
conv update, state update) must reproduce what ``forward`` over the longer prompt gives for that token
(tiled GEMMs, conv forward, scan)."""
import numpy as np
import pytest
import torch

from quamba_amd import W4A8QMamba, W4A8QMamba2, W8A8QMamba, W8A8QMamba2

pytestmark = pytest.mark.gpu


def _ri(dev, g, *shape, lo=-128, hi=128, dtype=torch.int8):
    return torch.randint(lo, hi, shape, dtype=dtype, device=dev, generator=g)


def _fill_linear(lin, dev, g, out_scale):
    """Random weights with scales that keep the int8 outputs inside the range without saturating everywhere."""
    if hasattr(lin, "s_group"):                               # 4-bit
        n, k = lin.size_n, lin.size_k
        lin.weight = _ri(dev, g, n, k // 2, lo=0, hi=256, dtype=torch.uint8)
        grouped = lin.s_group.numel() > 0
        if grouped:
            lin.s_group = (torch.rand(k // 128, n, device=dev, generator=g) * 13.8 + 2.0).half()
        # |acc| ~ 74 * 37 * sqrt(k) for grouped codes (|w8| up to 127), 74 * 64 * sqrt(k) per-channel
        lin.s_channel = torch.full((1, n), float(out_scale / (74.0 * (37.0 if grouped else 64.0) * np.sqrt(k))), device=dev)
        lin.input_scale = torch.tensor(1.0, device=dev)
    else:
        n, k = lin.out_features, lin.in_features
        lin._set_weight(_ri(dev, g, n, k))
        s = float(out_scale / (74.0 * 74.0 * np.sqrt(k)))
        lin.a = torch.tensor([[1.0]], device=dev)
        if lin.b.numel() > 1:
            lin.b = torch.full((1, lin.b.numel()), s, device=dev)
        else:
            lin.b = torch.tensor([[s]], dtype=torch.float32, device=dev)
        if hasattr(lin, "alpha"):
            lin.alpha = s


def _mamba1(cls, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    m = cls(256, 16, 4, device=dev, state_dtype=torch.float32)
    D, N = m.d_inner, m.d_state
    for lin in (m.in_proj, m.x_proj, m.dt_proj):
        _fill_linear(lin, dev, g, 40.0)
    _fill_linear(m.out_proj, dev, g, 1.0)
    m.conv1d.weight, m.conv1d.bias = _ri(dev, g, D, 4), _ri(dev, g, D)
    m.conv1d.input_scale, m.conv1d.weight_scale, m.conv1d.bias_scale, m.conv1d.output_scale = 0.04, 0.004, 0.004, 0.03
    sc = m.selective_scan
    sc.A_log, sc.D, sc.dt_bias = _ri(dev, g, D, N), _ri(dev, g, D), _ri(dev, g, D)
    for name, v in (("A_scale", 0.02), ("D_scale", 0.008), ("dt_bias_scale", 0.01), ("u_scale", 0.03), ("dt_scale", 0.02),
                    ("B_scale", 0.03), ("C_scale", 0.03), ("z_scale", 0.04), ("ssm_state_scale", 0.05)):
        setattr(sc, name, torch.tensor(v, device=dev))
    m.had.x_H_scale = 0.02
    return m, g


def _mamba2(cls, dev, seed):
    g = torch.Generator(device=dev).manual_seed(seed)
    G = 2
    m = cls(256, 64, 4, 2, 64, ngroups=G, chunk_size=64, device=dev, state_dtype=torch.float32, x_nhead_group=2, x_ndim_group=2)
    _fill_linear(m.in_proj, dev, g, 40.0)
    _fill_linear(m.out_proj, dev, g, 1.0)
    c = m.conv1d
    dim = c.weight.shape[0]
    c.weight, c.bias = _ri(dev, g, dim, 4), _ri(dev, g, dim)
    c.x_scale = c.B_scale = c.C_scale = 0.03
    c.wx_scale = c.wB_scale = c.wC_scale = 0.004
    c.bx_scale = c.bB_scale = c.bC_scale = 0.002
    c.x_out_scales = torch.rand(G, 2, 2, device=dev, generator=g) * 0.01 + 0.015
    c.B_out_scales = torch.tensor([0.02, 0.022], device=dev)
    c.C_out_scales = torch.tensor([0.021, 0.019], device=dev)
    c.x_head_group_range = torch.tensor([[1, 4], [3, 4]], dtype=torch.int32, device=dev)
    c.x_dim_group_range = torch.tensor([[[16, 64], [40, 64]], [[8, 64], [32, 64]]], dtype=torch.int32, device=dev)
    q = m.qchunk_scan
    q.A_log, q.D = _ri(dev, g, m.nheads, lo=0, hi=100), _ri(dev, g, m.nheads)
    q.dt_bias = torch.full((m.nheads,), -3.0, dtype=torch.float16, device=dev)
    q.A_log_scale, q.D_scale, q.dt_scale = (torch.tensor(v, device=dev) for v in (0.028, 0.008, 0.03))
    q.x_scales, q.B_scale, q.C_scale = c.x_out_scales, c.B_out_scales, c.C_out_scales
    q.x_head_group_range, q.x_dim_group_range = c.x_head_group_range, c.x_dim_group_range
    q.ssm_state_scale = torch.full((G, 2, 2, 64), 0.05, device=dev)
    m.norm.weight = (1 + 0.2 * torch.randn(m.d_ssm, device=dev, generator=g)).half()
    m.norm.z_scale = 0.03
    m.had.x_H_scale = 0.04
    return m, g


@pytest.mark.parametrize("cls,build", [(W4A8QMamba, _mamba1), (W8A8QMamba, _mamba1), (W8A8QMamba2, _mamba2), (W4A8QMamba2, _mamba2)])
def test_step_continues_forward(dev, cls, build):
    m, g = build(cls, dev, seed=3)
    B, L = 3, 70
    h = _ri(dev, g, B, L + 1, 256)
    full = m.forward(h)                                        # (B, L+1, d_model) fp16
    assert full.shape == (B, L + 1, 256) and full.dtype == torch.float16
    assert float(full.float().abs().max()) > 0 and bool(torch.isfinite(full.float()).all())
    conv_state, ssm_state = m.allocate_inference_cache(B)
    head = m.forward(h[:, :L].contiguous(), conv_state=conv_state, ssm_state=ssm_state)
    scale = float(full.float().abs().max())
    # a prefix of the prompt gives a prefix of the result (int8 stages are identical, fp16 stages to rounding)
    assert float((head.float() - full[:, :L].float()).abs().max()) <= 2e-2 * scale
    out, _, _ = m.step(h[:, L:L + 1].contiguous(), conv_state, ssm_state)
    diff = (out[:, 0].float() - full[:, L].float()).abs()
    # the Hadamard op quantises to int8 in between, so single values may move by one step: bound the bulk tightly
    assert float(diff.max()) <= 6e-2 * scale and float(diff.mean()) <= 5e-3 * scale
