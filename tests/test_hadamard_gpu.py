"""GPU parity of the Hadamard + int8 quantisation kernel against the CPU oracle: bit-exact (both sides
evaluate the same fp32 butterflies and left-to-right sums)."""
import math

import numpy as np
import pytest
import torch

import oracle
from quamba_amd import QHadamard, ops

pytestmark = pytest.mark.gpu


def _rows(rows, dim, seed, outliers=True):
    g = np.random.default_rng(seed)
    x = g.standard_normal((rows, dim)).astype(np.float32) * 2.0
    if outliers:
        cols = g.choice(dim, size=max(1, dim // 100), replace=False)
        x[:, cols] *= 20.0
    return x.astype(np.float16)


# model widths: 130m (12 * 128), 2.8b (40 * 128), Mamba2-8b (2^13), plus small and extreme forms
DIMS = [1536, 5120, 8192, 8, 16, 12, 40, 96, 640, 256, 4096, 32768, 12288]


@pytest.mark.parametrize("dim", DIMS)
def test_fp16_rows_bit_exact(dev, dim):
    x = _rows(7, dim, seed=dim)
    scale = np.float32(1.0 / math.sqrt(dim) / 0.06)
    want = oracle.hadamard_quant(x, scale)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale))
    assert got.dtype == torch.int8 and got.shape == x.shape
    np.testing.assert_array_equal(got.cpu().numpy(), want)
    assert np.abs(want).max() > 60


@pytest.mark.parametrize("dim", [1536, 5120, 8192, 2560, 12288])
def test_many_rows_take_the_one_lane_per_column_path(dev, dim):
    """More than 128 rows: 128 lanes per row, a lane produces all outputs of its column (few rows use
    four lanes per column).  The oracle is only run on a sample of the rows to keep the test short."""
    rows = 200
    x = _rows(rows, dim, seed=dim + 1)
    scale = np.float32(1.0 / math.sqrt(dim) / 0.06)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale)).cpu().numpy()
    pick = np.array([0, 1, 63, 128, 199])
    np.testing.assert_array_equal(got[pick], oracle.hadamard_quant(x[pick], scale))
    few = ops.hadamard_quant(torch.from_numpy(x[:100]).to(dev), float(scale)).cpu().numpy()
    np.testing.assert_array_equal(got[:100], few)


@pytest.mark.parametrize("dim", [2048, 4096, 8192])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_many_power_of_two_rows_take_the_32_values_per_lane_path(dev, dim, dtype):
    """More than 128 aligned rows of 2048, 4096 or 8192 columns: eight LDS planes, two round trips.  Same
    bits as the oracle, whose rows are a sample to keep the test short, and as the general kernel that
    rows off the 16-byte grid fall back to."""
    rows = 261
    x = _rows(rows, dim, seed=dim + 2).astype(dtype)
    scale = np.float32(1.0 / math.sqrt(dim) / 0.06)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale)).cpu().numpy()
    pick = np.array([0, 1, 127, 128, 129, 260])
    np.testing.assert_array_equal(got[pick], oracle.hadamard_quant(x[pick], scale))
    assert np.abs(got).max() > 60
    shifted = torch.zeros((rows, dim + 8), dtype=torch.from_numpy(x).dtype, device=dev)
    shifted[:, 1:dim + 1] = torch.from_numpy(x).to(dev)
    np.testing.assert_array_equal(ops.hadamard_quant(shifted[:, 1:dim + 1], float(scale)).cpu().numpy(), got)


@pytest.mark.parametrize("dim", [1536, 3072, 5120, 10240])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_many_rows_of_12_or_40_times_128_or_256_columns_take_the_lane_per_column_path(dev, dim, dtype):
    """More than 128 aligned rows of S * 128 or S * 256 columns: compile-time addressing, the S-point sums
    quantised in registers.  Same bits as the oracle (a sample of the rows) and as the general kernel that
    rows off the 16-byte grid fall back to."""
    rows = 197
    x = _rows(rows, dim, seed=dim + 3).astype(dtype)
    scale = np.float32(1.0 / math.sqrt(dim) / 0.06)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale)).cpu().numpy()
    pick = np.array([0, 1, 64, 127, 128, 196])
    np.testing.assert_array_equal(got[pick], oracle.hadamard_quant(x[pick], scale))
    assert np.abs(got).max() > 60
    shifted = torch.zeros((rows, dim + 8), dtype=torch.from_numpy(x).dtype, device=dev)
    shifted[:, 1:dim + 1] = torch.from_numpy(x).to(dev)
    np.testing.assert_array_equal(ops.hadamard_quant(shifted[:, 1:dim + 1], float(scale)).cpu().numpy(), got)


@pytest.mark.parametrize("rows,dim", [(2100, 8192), (4173, 2048)])
def test_more_rows_than_resident_workgroups(dev, rows, dim):
    """The 32-values-per-lane kernel launches as many workgroups as the chip holds and lets each walk several
    rows with the next row's loads in flight: first, middle and last rows of such walks against the oracle."""
    x = _rows(rows, dim, seed=rows)
    scale = np.float32(1.0 / math.sqrt(dim) / 0.06)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale)).cpu().numpy()
    pick = np.array([0, 1, 1023, 1024, 1025, 2047, 2048, 2049, rows - 2, rows - 1])
    np.testing.assert_array_equal(got[pick], oracle.hadamard_quant(x[pick], scale))
    # every row: the same bytes as when the row is transformed in a small call of its own
    few = ops.hadamard_quant(torch.from_numpy(x[1000:1100]).to(dev), float(scale)).cpu().numpy()
    np.testing.assert_array_equal(got[1000:1100], few)
    tail = ops.hadamard_quant(torch.from_numpy(x[-150:]).to(dev), float(scale)).cpu().numpy()
    np.testing.assert_array_equal(got[-150:], tail)


def test_rounding_at_ties_and_saturation_on_the_32_values_per_lane_path(dev):
    """Rows whose transform lands exactly on k + 1/2 and beyond the int8 range: half away from zero, then
    saturation, as the general kernel does."""
    dim, rows = 2048, 256
    x = np.zeros((rows, dim), dtype=np.float16)
    x[:, 0] = (np.arange(rows) - 128).astype(np.float16) * 0.5 + 0.25      # every output of row r is x[r, 0]
    x[200:, 0] *= 8.0
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), 2.0).cpu().numpy()
    want = oracle.hadamard_quant(x, np.float32(2.0))
    np.testing.assert_array_equal(got, want)
    assert want.min() == -128 and want.max() == 127 and (np.abs(2.0 * x[:200, 0].astype(np.float32)) % 1 == 0.5).all()


def test_fp32_input_and_leading_dims(dev):
    x = _rows(24, 5120, seed=3).astype(np.float32).reshape(2, 12, 5120)
    scale = np.float32(1.0 / math.sqrt(5120) / 0.05)
    want = oracle.hadamard_quant(x, scale)
    got = ops.hadamard_quant(torch.from_numpy(x).to(dev), float(scale))
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_strided_rows(dev):
    x = _rows(9, 1536, seed=5)
    buf = torch.zeros((9, 2048), dtype=torch.float16, device=dev)
    buf[:, :1536] = torch.from_numpy(x).to(dev)
    want = oracle.hadamard_quant(x, 0.4)
    got = ops.hadamard_quant(buf[:, :1536], 0.4)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_module_folds_scales_and_keeps_state(dev):
    dim = 5120
    m = QHadamard(dim, x_H_scale=0.043)
    assert m.N == 40 and abs(m.had_scale - 1 / math.sqrt(dim)) < 1e-12
    x = _rows(5, dim, seed=8)
    want = oracle.hadamard_quant(x, np.float32(m.had_scale / 0.043))
    np.testing.assert_array_equal(m(torch.from_numpy(x).to(dev)).cpu().numpy(), want)
    m2 = QHadamard(dim)
    m2.load_state_dict(m.state_dict())
    assert m2.x_H_scale == pytest.approx(0.043)
    assert QHadamard(1536).N == 12 and QHadamard(8192).N == 2


def test_rotation_preserves_the_linear_layer(dev):
    # (H x / sqrt(d)) . (H w / sqrt(d)) == x . w : what makes the rotated out_proj equivalent
    dim = 1536
    g = np.random.default_rng(0)
    x = g.standard_normal((3, dim)).astype(np.float16)
    w = g.standard_normal((3, dim)).astype(np.float16)
    s = 24.0 / math.sqrt(dim)       # int8 grid of 1/24 over +-5.3: no saturation for unit-variance rows
    hx = ops.hadamard_quant(torch.from_numpy(x).to(dev), s).float() / 24.0
    hw = ops.hadamard_quant(torch.from_numpy(w).to(dev), s).float() / 24.0
    want = (torch.from_numpy(x).float() * torch.from_numpy(w).float()).sum(-1)
    assert torch.allclose((hx * hw).sum(-1).cpu(), want, atol=3.0)      # rounding noise ~ sqrt(dim) * 0.017


def test_unsupported_width(dev):
    with pytest.raises(NotImplementedError):
        ops.hadamard_quant(torch.zeros((2, 24 * 5), dtype=torch.float16, device=dev), 1.0)
