"""Pins the CPU oracle's W8A8 GEMM restatement (no GPU): exact integer matmul, epilogue order and
rounding, written independently with numpy."""
import numpy as np

import oracle


def test_accumulators_equal_integer_matmul_and_epilogue_order():
    g = np.random.default_rng(1)
    M, N, K = 37, 29, 208
    a = g.integers(-128, 128, (M, K)).astype(np.int8)
    w = g.integers(-128, 128, (N, K)).astype(np.int8)
    sa = g.uniform(0.001, 0.01, M).astype(np.float32)
    sb = g.uniform(0.001, 0.01, N).astype(np.float32)
    acc, f, q = oracle.gemm_w8a8(a, w, sa, sb)
    want_acc = a.astype(np.int64) @ w.astype(np.int64).T
    np.testing.assert_array_equal(acc, want_acc)
    want_f = sa[:, None] * (sb[None, :] * want_acc.astype(np.float32))       # fp32, this association
    np.testing.assert_array_equal(f, want_f)
    np.testing.assert_array_equal(q, np.clip(np.rint(want_f), -128, 127).astype(np.int8))
    # per-tensor scales broadcast
    _, f1, _ = oracle.gemm_w8a8(a, w, sa[:1], sb[:1])
    np.testing.assert_array_equal(f1, sa[0] * (sb[0] * want_acc.astype(np.float32)))
    # extreme operands do not overflow int32 for K this size
    a[:] = -128
    w[:] = -128
    acc, _, _ = oracle.gemm_w8a8(a, w, sa, sb)
    assert (acc == 128 * 128 * K).all()


def test_rounding_modes_on_exact_halves():
    # acc * 0.5 lands on x.5: RNE goes to even, the GEMV rule goes away from zero
    a = np.array([[1, 3, 5, -1, -3, 127]], np.int8).T.copy()      # (6,1) rows
    a = np.pad(a, ((0, 0), (0, 15)))
    w = np.zeros((1, 16), np.int8)
    w[0, 0] = 1
    one, half = np.float32([1.0]), np.float32([0.5])
    _, _, q_rne = oracle.gemm_w8a8(a, w, one, half)
    _, _, q_away = oracle.gemm_w8a8(a, w, one, half, round_half_away=True)
    np.testing.assert_array_equal(q_rne[:, 0], [0, 2, 2, 0, -2, 64])
    np.testing.assert_array_equal(q_away[:, 0], [1, 2, 3, -1, -2, 64])
    _, _, q_sat = oracle.gemm_w8a8(a, w, np.float32([4.0]), one)
    np.testing.assert_array_equal(q_sat[:, 0], [4, 12, 20, -4, -12, 127])
