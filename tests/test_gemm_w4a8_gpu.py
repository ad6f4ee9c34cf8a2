"""GPU parity of the W4A8 GEMM and linear modules against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import W4A8B8O8Linear, W4A8B8O8LinearParallel, W4A8B16O16Linear, ops
from quamba_amd import w4a8_utils as wu

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _case(M, N, K, seed, grouped=True):
    g = np.random.default_rng(seed)
    a = g.integers(-128, 128, (M, K)).astype(np.int8)
    if grouped:
        codes = g.integers(0, 16, (N, K)).astype(np.uint8)
        sg = g.uniform(2.0, 15.8, (K // 128, N)).astype(np.float16)
    else:
        codes = (g.integers(-7, 8, (N, K)) & 0xF).astype(np.uint8)
        sg = None
    sc = (g.uniform(0.5, 1.5, N) * 0.06 / np.sqrt(K) / 8).astype(np.float32)
    st = g.uniform(0.5, 1.5, M).astype(np.float32)
    return a, codes, sg, sc, st


def _run(dev, a, codes, sg, sc, st, out8, transpose=False, per_token=True):
    M, K = a.shape
    N = codes.shape[0]
    packed = wu.pack_w4a8(torch.from_numpy(codes.T.astype(np.int32)))
    fn = ops.w4a8o8_gemm if out8 else ops.w4a8o16_gemm
    s_tok = _t(st if per_token else st[:1], dev)
    return fn(_t(a, dev), packed.to(dev), s_tok, _t(sc[None], dev), None if sg is None else _t(sg, dev),
              None, M, N, K, transpose)


SHAPES = [(256, 256, 128), (300, 200, 384), (17, 70, 256), (1, 64, 128), (2048, 1024, 512), (4096, 4160, 1024),
          # few rows (the decode step's kernel): one and two row blocks, K split over four and eight waves,
          # a K that ends in the middle of a 256-code piece, fewer pieces than waves
          (1, 4096, 8192), (33, 100, 4224), (64, 9000, 1280), (5, 200, 384), (65, 96, 4096)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("grouped", [True, False])
def test_int8_output_bit_exact(dev, M, N, K, grouped):
    a, codes, sg, sc, st = _case(M, N, K, M + N + K, grouped)
    _, _, _, want = oracle.gemm_w4a8(a, codes, sg, sc, st)
    got = _run(dev, a, codes, sg, sc, st, out8=True)
    assert got.shape == (M, N)
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    assert np.abs(want).max() > 20


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 384), (2048, 1024, 512), (64, 520, 4352), (3, 70, 640)])
def test_fp16_and_transposed_outputs_bit_exact(dev, M, N, K):
    a, codes, sg, sc, st = _case(M, N, K, 7 * M + K)
    _, _, f, q = oracle.gemm_w4a8(a, codes, sg, sc, st[:1])
    got = _run(dev, a, codes, sg, sc, st, out8=False, per_token=False)
    np.testing.assert_array_equal(got.cpu().numpy(), f.astype(np.float16))
    got_t = _run(dev, a, codes, sg, sc, st, out8=False, transpose=True, per_token=False)
    assert got_t.shape == (N, M)
    np.testing.assert_array_equal(got_t.cpu().numpy(), f.astype(np.float16).T)
    got_t8 = _run(dev, a, codes, sg, sc, st, out8=True, transpose=True, per_token=False)
    np.testing.assert_array_equal(got_t8.cpu().numpy(), q.T)


def _linear(out_f, in_f, seed, dev):
    lin = torch.nn.Linear(in_f, out_f, bias=False, dtype=torch.float16)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(out_f, in_f, generator=g) / in_f ** 0.5).half())
    return lin.to(dev)


def test_w4a8_linears_match_oracle_and_track_the_fp_layer(dev):
    in_f, out_f, B, L = 256, 200, 3, 37                      # out pads to 256
    lin = _linear(out_f, in_f, 1, dev)
    x_f = torch.randn(B, L, in_f, device=dev)
    s_in = x_f.abs().max() / 127
    x = torch.clamp(torch.round(x_f / s_in), -128, 127).to(torch.int8)

    q16 = W4A8B16O16Linear.from_fp16(lin, s_in)
    assert q16.weight.dtype == torch.uint8 and q16.weight.shape == (256, in_f // 2)
    assert q16.s_group.shape == (2, 256) and q16.s_channel.shape == (1, 256) and q16.input_scale.shape == ()
    assert set(q16.state_dict()) == {"workspace", "weight", "input_scale", "s_channel", "s_group"}
    y = q16(x)
    assert y.shape == (B, L, out_f) and y.dtype == torch.float16
    codes = wu.unpack_w4a8(q16.weight.cpu()).numpy().T.astype(np.uint8)           # (N, K)
    _, _, f, _ = oracle.gemm_w4a8(x.view(-1, in_f).cpu().numpy(), codes, q16.s_group.cpu().numpy(),
                                  q16.s_channel.cpu().numpy(), q16.input_scale.cpu().numpy())
    np.testing.assert_array_equal(y.cpu().numpy().reshape(-1, out_f), f.astype(np.float16)[:, :out_f])
    # reference acceptance test: against the linear layer built from the dequantised weights w_ref
    ref = (x.float() * s_in) @ q16.w_ref[:, :out_f].float().to(dev)
    r2 = ((y.float() - ref) ** 2).sum() / (ref ** 2).sum()
    assert r2 < 1e-3 and (y.float() - ref).abs().max() < 0.1
    yt = q16.to_seqlen_last(x)
    assert yt.shape == (B, out_f, L) and yt.stride(2) == 1
    assert torch.equal(yt.transpose(1, 2), y)

    s_out = ref.abs().max() / 127
    q8 = W4A8B8O8Linear.from_fp16(lin, s_in, s_out)
    y8 = q8(x)
    assert y8.dtype == torch.int8
    _, _, _, q = oracle.gemm_w4a8(x.view(-1, in_f).cpu().numpy(), wu.unpack_w4a8(q8.weight.cpu()).numpy().T.astype(np.uint8),
                                  q8.s_group.cpu().numpy(), q8.s_channel.cpu().numpy(), q8.input_scale.cpu().numpy())
    np.testing.assert_array_equal(y8.cpu().numpy().reshape(-1, out_f), q[:, :out_f])
    rel = ((y8.float() * s_out - ref).abs().mean() / ref.abs().mean()).item()
    assert rel < 0.08                                          # the reference's bound for the int8 output
    assert torch.equal(q8.to_seqlen_last(x).transpose(1, 2), y8)

    qp = W4A8B8O8LinearParallel.from_fp16(lin, s_in, [s_out, 2 * s_out], [120, 80])
    yp = qp(x)
    assert torch.equal(yp[..., :120], y8[..., :120])
    rel = ((yp[..., 120:].float() * 2 * s_out - ref[..., 120:]).abs().mean() / ref[..., 120:].abs().mean()).item()
    assert rel < 0.095


def test_small_in_features_use_per_channel_mode(dev):
    lin = _linear(64, 128, 5, dev)
    x = torch.randint(-128, 128, (4, 9, 128), dtype=torch.int8, device=dev)
    q = W4A8B16O16Linear.from_fp16(lin, torch.tensor(0.01))
    assert q.s_group.numel() == 0
    y = q(x)
    ref = (x.float() * 0.01) @ q.w_ref.float().to(dev)
    torch.testing.assert_close(y.float(), ref, rtol=2e-3, atol=2e-3)


def test_errors(dev):
    a = torch.zeros((8, 64), dtype=torch.int8, device=dev)
    w = torch.zeros((16, 32), dtype=torch.uint8, device=dev)
    one = torch.ones(1, device=dev)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ops.w4a8o16_gemm(a, w, one, torch.ones(16, device=dev), None, None, 8, 16, 64)


def test_reference_checkpoint_loads_and_computes_the_same(dev):
    """A state dict in the reference module's own format (Marlin-QQQ int32 weight, permuted scales, lock
    workspace; vectors from the reference's packer in tests/golden) loads into the module here and gives
    the same output as the layer quantised natively from the same fp16 weight."""
    import os
    fix = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "marlin_qqq_w4a8.npz"))
    K, N = 256, 128
    ref_sd = {"workspace": torch.zeros((N // 64) * 16, dtype=torch.int32),
              "weight": torch.from_numpy(fix["g_marlin_q_w"]),
              "input_scale": torch.tensor(0.02),
              "s_channel": torch.from_numpy(fix["g_marlin_s_channel"]),
              "s_group": torch.from_numpy(fix["g_marlin_s_group"])}
    m = W4A8B16O16Linear(K, N, device=dev)
    m.load_state_dict(ref_sd)
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
    lin.weight.data = torch.from_numpy(fix["g_w"]).t().contiguous()
    native = W4A8B16O16Linear.from_fp16(lin.to(dev), torch.tensor(0.02))
    assert torch.equal(m.weight, native.weight) and torch.equal(m.s_group, native.s_group)
    x = torch.randint(-128, 128, (3, 50, K), dtype=torch.int8, device=dev)
    assert torch.equal(m(x), native(x))
    assert m(x).float().abs().max() > 0.1


@pytest.mark.parametrize("grouped", [True, False])
@pytest.mark.parametrize("out8", [True, False])
def test_expanding_the_weights_once_gives_the_same_bits(dev, monkeypatch, grouped, out8):
    """With a scratch buffer the weights are expanded to int8 once and the int8 x int8 kernel runs on them;
    the wrapper only passes the buffer for large products, so the threshold is lowered here."""
    M, N, K = 300, 520, 512
    a, codes, sg, sc, st = _case(M, N, K, seed=9, grouped=grouped)
    fused = _run(dev, a, codes, sg, sc, st, out8)
    monkeypatch.setattr(ops, "W4A8_EXPAND_ONCE_ROWS", 0)
    once = _run(dev, a, codes, sg, sc, st, out8)
    assert torch.equal(fused, once)
    per_tensor = _run(dev, a, codes, sg, sc, st, out8, per_token=False)
    once_t = _run(dev, a, codes, sg, sc, st, out8, transpose=True)         # (N, M): the operands' roles exchanged
    assert once_t.shape == (N, M) and torch.equal(once_t.t(), once)
    monkeypatch.setattr(ops, "W4A8_EXPAND_ONCE_ROWS", 1 << 30)
    assert torch.equal(per_tensor, _run(dev, a, codes, sg, sc, st, out8, per_token=False))
    assert torch.equal(once_t, _run(dev, a, codes, sg, sc, st, out8, transpose=True))
