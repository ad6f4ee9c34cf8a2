"""Empty inputs (no batch entries, no steps, no rows) through every operator: each returns tensors of the right
shapes and types without a launch and without an error, and leaves a carried state as it was."""
import numpy as np
import pytest
import torch

from quamba_amd import QRMSNormGated, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _s(v, dev):
    return torch.tensor([float(v)], dtype=torch.float32, device=dev)


@pytest.mark.parametrize("B,L", [(0, 16), (2, 0)])
def test_conv_forward(dev, B, L):
    D, k = 64, 4
    qw, sw, qb, sb = synth.conv_weights(D, k, 1)
    x = torch.zeros((B, D, L), dtype=torch.int8, device=dev)
    out = ops.causal_conv1d_fwd(x, 0.02, _t(qw, dev), sw, 0.03, sb, _t(qb, dev))
    assert out.shape == (B, D, L) and out.dtype == torch.int8
    out, out_t = ops.causal_conv1d_fwd(x, 0.02, _t(qw, dev), sw, 0.03, sb, _t(qb, dev), also_channel_last=True)
    assert out.shape == (B, D, L) and out_t.shape == (B, L, D)


def test_conv_update_without_batch_entries(dev):
    D, k = 64, 4
    qw, sw, qb, sb = synth.conv_weights(D, k, 1)
    x = torch.zeros((0, D), dtype=torch.int8, device=dev)
    state = torch.zeros((0, D, k), dtype=torch.int8, device=dev)
    out = ops.causal_conv1d_update(x, state, 0.02, _t(qw, dev), sw, 0.03, sb, _t(qb, dev))
    assert out.shape == (0, D) and out.dtype == torch.int8


@pytest.mark.parametrize("B,L", [(0, 16), (2, 0)])
@pytest.mark.parametrize("N", [16, 64])
def test_selective_scan_forward(dev, B, L, N):
    D = 64
    d = synth.mamba1_scan_inputs(1, 8, D, N, seed=3)
    z8 = lambda *s: torch.zeros(s, dtype=torch.int8, device=dev)
    y, state = ops.sscan_fwd(z8(B, D, L), _s(d["s_u"], dev), z8(B, D, L), _s(d["s_dt"], dev), _t(d["A_log"], dev), _s(d["s_A"], dev),
                             z8(B, 1, N, L), _s(d["s_B"], dev), z8(B, 1, N, L), _s(d["s_C"], dev), _s(0.05, dev),
                             _t(d["D"], dev), _s(d["s_D"], dev), z8(B, D, L), _s(0.02, dev), _t(d["dt_bias"], dev), _s(d["s_db"], dev),
                             True, state_dtype=torch.float32)
    assert y.shape == (B, L, D) and y.dtype == torch.float16
    assert state.shape[0] == B and state.shape[1] == D and state.shape[-1] == N
    if B > 0:
        # no steps: the state after the last step is the zero state the scan starts from
        assert float(state.float().abs().max()) == 0.0


@pytest.mark.parametrize("B,L", [(0, 100), (2, 0)])
@pytest.mark.parametrize("P,N,Q", [(64, 128, 64), (96, 48, 100)])
def test_ssd_chunk_scan(dev, B, L, P, N, Q):
    H, G = 4, 2
    d = synth.mamba2_ssd_inputs(1, 8, H, P, N, G, seed=2)
    z8 = lambda *s: torch.zeros(s, dtype=torch.int8, device=dev)
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    y, final = ops.ssd_chunk_scan_combined_fwd(z8(B, L, H, P), s(d["x_scale"]), z8(B, L, H), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
                                               z8(B, L, G, N), s(d["s_B"]), z8(B, L, G, N), s(d["s_C"]), None, Q,
                                               q_D=_t(d["D"], dev), D_scale=s(d["s_D"]), dt_bias=_t(d["dt_bias"], dev),
                                               dt_softplus=True, final_state_dtype=torch.float32)
    assert y.shape == (B, L, H, P) and y.dtype == torch.float16 and final.shape == (B, H, P, N)


@pytest.mark.parametrize("dim", [5120, 8192, 96])
def test_hadamard_without_rows(dev, dim):
    out = ops.hadamard_quant(torch.zeros((0, dim), dtype=torch.float16, device=dev), 0.5)
    assert out.shape == (0, dim) and out.dtype == torch.int8
    out = ops.hadamard_quant(torch.zeros((2, 0, dim), dtype=torch.float16, device=dev), 0.5)
    assert out.shape == (2, 0, dim)


@pytest.mark.parametrize("f16", [True, False])
def test_gated_norm_without_rows(dev, f16):
    N = 256
    m = QRMSNormGated(N, eps=1e-5, group_size=64, norm_before_gate=True, use_float16_output=f16, device=dev)
    m.z_scale, m.output_scale = 0.02, 0.05
    x = torch.zeros((0, N), dtype=torch.float16, device=dev)
    out = m(x, torch.zeros((0, N), dtype=torch.int8, device=dev))
    out = out[0] if isinstance(out, tuple) else out
    assert out.shape == (0, N) and out.dtype == (torch.float16 if f16 else torch.int8)


@pytest.mark.parametrize("M,N", [(0, 64), (16, 0)])
def test_w8a8_gemm(dev, M, N):
    K = 128
    a = torch.zeros((M, K), dtype=torch.int8, device=dev)
    w = torch.zeros((N, K), dtype=torch.int8, device=dev)
    for dtype in (torch.int8, torch.float16):
        c = torch.empty((M, N), dtype=dtype, device=dev)
        ops.scaled_mm_dq(c, a, w.t(), torch.ones(1, device=dev), torch.ones(1, device=dev))
        assert c.shape == (M, N)


def test_w4a8_gemm_without_rows(dev):
    N, K = 64, 256
    a = torch.zeros((0, K), dtype=torch.int8, device=dev)
    wq = torch.zeros((N, K // 2), dtype=torch.uint8, device=dev)
    s_ch = torch.ones(N, dtype=torch.float32, device=dev)
    s_tok = torch.ones(1, dtype=torch.float32, device=dev)
    s_group = torch.ones((K // 128, N), dtype=torch.float16, device=dev)
    out = ops.w4a8o16_gemm(a, wq, s_tok, s_ch, s_group, None, 0, N, K)
    assert out.shape == (0, N) and out.dtype == torch.float16
    out = ops.w4a8o8_gemm(a, wq, s_tok, s_ch, s_group, None, 0, N, K)
    assert out.shape == (0, N) and out.dtype == torch.int8
