"""GPU parity of the W8A8 GEMM and the linear modules against the CPU oracle: int8 outputs and
fp16 outputs bit-exact (integer accumulation is exact and the epilogue is IEEE fp32)."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import W8A8B8O8Linear, W8A8B8O8LinearParallel, W8A8B16O16Linear, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _operands(M, N, K, seed):
    g = np.random.default_rng(seed)
    a = g.integers(-128, 128, (M, K)).astype(np.int8)
    w = g.integers(-128, 128, (N, K)).astype(np.int8)
    # scales sized so outputs span the int8 range without saturating everywhere
    sa = (g.uniform(0.5, 1.5, M) * 0.4 / np.sqrt(K)).astype(np.float32)
    sb = (g.uniform(0.5, 1.5, N) * 0.02).astype(np.float32)
    return a, w, sa, sb


# (M, N, K): tile-aligned, ragged in every dimension, tiny, single row, big-tile path
SHAPES = [(256, 256, 128), (128, 128, 64), (300, 200, 208), (1, 48, 64), (17, 33, 16), (70, 1000, 1536),
          (2048, 4096, 256), (4096, 4112, 320), (64, 16, 2560),
          # few rows (the decode step's kernel): one and two row blocks, K split over four and eight waves,
          # a K that ends inside a 32-byte step, fewer K tiles than waves
          (33, 100, 5120), (5, 200, 2064), (64, 5120, 160), (1, 2560, 5120), (32, 10240, 2560), (65, 96, 4096),
          # few 128x128 tiles and a long K: the four-stage form of the small tile, K ending inside a tile
          (130, 136, 1104), (1000, 192, 5120),
          # one round of 320x256 tiles where 256x256 tiles would need two: whole tiles, and ragged in both directions
          (2560, 8192, 64), (2400, 8100, 80)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("per_row,per_col", [(False, False), (True, True), (False, True)])
def test_int8_output_bit_exact(dev, M, N, K, per_row, per_col):
    a, w, sa, sb = _operands(M, N, K, seed=M + N + K)
    sa = sa if per_row else sa[:1]
    sb = sb if per_col else sb[:1]
    _, _, want = oracle.gemm_w8a8(a, w, sa, sb)
    c = torch.empty((M, N), dtype=torch.int8, device=dev)
    ops.scaled_mm_dq(c, _t(a, dev), _t(w, dev).t(), _t(sa, dev), _t(sb, dev))
    got = c.cpu().numpy()
    np.testing.assert_array_equal(got, want)
    assert np.abs(want).max() > 20


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 208), (33, 24, 48), (2048, 2560, 512),
                                   (64, 2560, 5120), (7, 50, 4112)])
def test_fp16_output_bit_exact(dev, M, N, K):
    a, w, sa, sb = _operands(M, N, K, seed=3 * M + K)
    _, f, _ = oracle.gemm_w8a8(a, w, sa[:1], sb)
    c = torch.empty((M, N), dtype=torch.float16, device=dev)
    ops.scaled_mm_dq(c, _t(a, dev), _t(w, dev).t(), _t(sa[:1], dev), _t(sb, dev))
    np.testing.assert_array_equal(c.cpu().numpy(), f.astype(np.float16))


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 200, 208), (33, 24, 48), (2048, 2560, 512),
                                   (64, 2560, 5120), (1, 48, 64), (2400, 8100, 80)])
def test_bf16_output_bit_exact(dev, M, N, K):
    """bf16 = the oracle's fp32 value rounded to nearest even (the reference's converter); compared as bit patterns."""
    a, w, sa, sb = _operands(M, N, K, seed=5 * M + K)
    _, f, _ = oracle.gemm_w8a8(a, w, sa, sb)
    c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    ops.scaled_mm_dq(c, _t(a, dev), _t(w, dev).t(), _t(sa, dev), _t(sb, dev))
    u = np.ascontiguousarray(f, np.float32).view(np.uint32).astype(np.uint64)
    want = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(want, torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))
    np.testing.assert_array_equal(c.view(torch.int16).cpu().numpy().view(np.uint16), want)


@pytest.mark.parametrize("out_dtype", [torch.int8, torch.float16])
def test_wide_tile_path_matches_exact_fp32(dev, out_dtype):
    """16384 x 2560 is the shape for which the 256x320 tile is chosen (two full rounds of workgroups).
    K = 256 keeps every integer sum below 2^24, so an fp32 matmul is exact and torch applies the same
    two IEEE multiplications; rounding to int8 is torch's round-half-even."""
    M, N, K = 16384, 2560, 256
    g = torch.Generator(device="cpu").manual_seed(5)
    a = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g).to(dev)
    w = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(dev)
    sa = (torch.rand(M, generator=g) * 0.02 + 0.01).to(dev)
    sb = (torch.rand(N, generator=g) * 0.02 + 0.01).to(dev)
    c = torch.empty((M, N), dtype=out_dtype, device=dev)
    ops.scaled_mm_dq(c, a, w.t(), sa, sb)
    acc = a.float() @ w.float().t()
    want = sa[:, None] * (sb[None, :] * acc)
    if out_dtype == torch.int8:
        want = torch.clamp(torch.round(want), -128, 127).to(torch.int8)
        assert want.abs().max().item() > 50
    else:
        want = want.half()
    assert torch.equal(c, want)


def test_output_with_row_padding(dev):
    M, N, K = 100, 72, 64
    a, w, sa, sb = _operands(M, N, K, seed=9)
    buf = torch.full((M, 96), 7, dtype=torch.int8, device=dev)
    c = buf[:, :N]
    ops.scaled_mm_dq(c, _t(a, dev), _t(w, dev).t(), _t(sa[:1], dev), _t(sb[:1], dev))
    np.testing.assert_array_equal(c.cpu().numpy(), oracle.gemm_w8a8(a, w, sa[:1], sb[:1])[2])
    assert (buf[:, N:] == 7).all()


def test_single_row_rules(dev):
    N, K = 272, 256
    a, w, sa, sb = _operands(1, N, K, seed=4)
    alpha = np.float32(0.0031)
    acc = oracle.gemm_w8a8(a, w, np.float32([1]), np.float32([1]))[0]
    y = torch.empty((1, N), dtype=torch.int8, device=dev)
    ops.scaled_mv_dq(y, _t(w, dev), _t(a, dev), float(alpha), 0.0)
    np.testing.assert_array_equal(y.cpu().numpy(), np.clip(np.rint(alpha * acc.astype(np.float32)), -128, 127))
    y16 = torch.empty((1, N), dtype=torch.float16, device=dev)
    ops.scaled_mv_dq(y16, _t(w, dev), _t(a, dev), float(alpha), 0.0)
    np.testing.assert_array_equal(y16.cpu().numpy(), (alpha * acc.astype(np.float32)).astype(np.float16))
    ops.w8a8o8_gemv(y, _t(w, dev), _t(a, dev), _t(sb[None], dev), _t(sa[:1, None], dev))
    want = oracle.gemm_w8a8(a, w, sa[:1], sb, round_half_away=True)[2]
    np.testing.assert_array_equal(y.cpu().numpy(), want)


def _linear(out_f, in_f, seed):
    lin = torch.nn.Linear(in_f, out_f, bias=False)
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        lin.weight.copy_(torch.randn(out_f, in_f, generator=g) / in_f ** 0.5)
    return lin


def test_w8a8b8o8_linear_forward_and_seqlen_last(dev):
    in_f, out_f, B, L = 256, 200, 3, 37                # out_f pads to 208; B*L = 111 pads to 112
    lin = _linear(out_f, in_f, 1).to(dev)
    q = W8A8B8O8Linear.from_fp16(lin, input_scale=0.02, output_scale=0.015)
    assert q.weight.shape == (in_f, 208) and q.weight.stride() == (1, in_f) and q.a.shape == (1, 1)
    sd = q.state_dict()
    assert set(sd) == {"weight", "a", "b", "alpha"}
    x = torch.randint(-128, 128, (B, L, in_f), dtype=torch.int8, device=dev)
    w_nk = q.weight.t().contiguous().cpu().numpy()[:out_f]
    want = oracle.gemm_w8a8(x.view(-1, in_f).cpu().numpy(), w_nk, q.a.cpu().numpy(), q.b.cpu().numpy())[2]
    y = q(x)
    assert y.shape == (B, L, out_f) and y.dtype == torch.int8
    np.testing.assert_array_equal(y.cpu().numpy().reshape(-1, out_f), want)
    yt = q.to_seqlen_last(x)
    assert yt.shape == (B, out_f, L) and yt.stride(2) == 1
    # the operands' roles swap (b scales the rows), the product a*(b*acc) keeps its association
    want_t = oracle.gemm_w8a8(w_nk, x.view(-1, in_f).cpu().numpy(), q.b.cpu().numpy(), q.a.cpu().numpy())[2]
    np.testing.assert_array_equal(yt.cpu().numpy(), want_t.reshape(out_f, B, L).transpose(1, 0, 2))
    y1 = q(x[:1, :1])
    acc = oracle.gemm_w8a8(x[0, :1].cpu().numpy(), w_nk, np.float32([1]), np.float32([1]))[0]
    np.testing.assert_array_equal(y1.cpu().numpy().reshape(1, -1),
                                  np.clip(np.rint(np.float32(q.alpha) * acc.astype(np.float32)), -128, 127))
    q2 = W8A8B8O8Linear(in_f, out_f, device=dev)
    q2.load_state_dict(sd)
    assert torch.equal(q2(x), y) and q2.alpha == q.alpha


def test_parallel_and_fp16_out_linears(dev):
    in_f, splits = 128, [96, 40, 24]
    lin = _linear(sum(splits), in_f, 2).to(dev)
    q = W8A8B8O8LinearParallel.from_fp16(lin, 0.02, [0.01, 0.02, 0.03], splits)
    assert q.b.shape == (1, 160)
    x = torch.randint(-128, 128, (2, 9, in_f), dtype=torch.int8, device=dev)
    w_nk = q.weight.t().contiguous().cpu().numpy()
    want = oracle.gemm_w8a8(x.view(-1, in_f).cpu().numpy(), w_nk, q.a.cpu().numpy(), q.b.cpu().numpy())[2]
    np.testing.assert_array_equal(q(x).cpu().numpy().reshape(-1, 160), want)
    want1 = oracle.gemm_w8a8(x[0, :1].cpu().numpy(), w_nk, q.a.cpu().numpy(), q.b.cpu().numpy(), round_half_away=True)[2]
    np.testing.assert_array_equal(q(x[:1, :1]).cpu().numpy().reshape(1, -1), want1)

    lin2 = _linear(100, in_f, 3).to(dev)
    q16 = W8A8B16O16Linear.from_fp16(lin2, input_scale=0.02)
    y = q16(x)
    assert y.dtype == torch.float16 and y.shape == (2, 9, 100)
    f = oracle.gemm_w8a8(x.view(-1, in_f).cpu().numpy(), q16.weight.t().contiguous().cpu().numpy()[:100],
                         q16.a.cpu().numpy(), q16.b.cpu().numpy())[1]
    np.testing.assert_array_equal(y.cpu().numpy().reshape(-1, 100), f.astype(np.float16))
    # dequantised result tracks the fp32 linear layer (the reference's own acceptance test)
    ref = (x.float() * 0.02) @ lin2.weight.float().t()
    r2 = ((y.float() - ref) ** 2).sum() / (ref ** 2).sum()
    assert r2 < 1e-3


def test_errors(dev):
    a = torch.zeros((16, 24), dtype=torch.int8, device=dev)       # K = 24 is not a multiple of 16
    w = torch.zeros((16, 24), dtype=torch.int8, device=dev)
    s = torch.ones(1, device=dev)
    with pytest.raises(RuntimeError, match="multiples of 16"):
        ops.scaled_mm_dq(torch.empty((16, 16), dtype=torch.int8, device=dev), a, w.t(), s, s)
    a = torch.zeros((16, 32), dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError, match="column-major"):
        ops.scaled_mm_dq(torch.empty((16, 16), dtype=torch.int8, device=dev), a, torch.zeros((32, 16), dtype=torch.int8, device=dev), s, s)
    with pytest.raises(RuntimeError, match="1 or 16"):
        ops.scaled_mm_dq(torch.empty((16, 16), dtype=torch.int8, device=dev), a, a.t(), torch.ones(3, device=dev), s)
