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


# ------------------------------------------------------------------------------------------------
# W4A8
# ------------------------------------------------------------------------------------------------
def _w4_case(M, N, K, seed):
    g = np.random.default_rng(seed)
    a = g.integers(-128, 128, (M, K)).astype(np.int8)
    codes = g.integers(0, 16, (N, K)).astype(np.uint8)
    sg = g.uniform(1.0, 15.0, (K // 128, N)).astype(np.float16)
    sc = g.uniform(1e-3, 2e-3, N).astype(np.float32)
    st = g.uniform(0.5, 1.5, M).astype(np.float32)
    return a, codes, sg, sc, st


def test_w4a8_unit_group_scale_is_a_pure_integer_gemm():
    a, codes, _, sc, st = _w4_case(9, 13, 256, 3)
    ones = np.ones((2, 13), np.float16)
    w8, acc, f, q = oracle.gemm_w4a8(a, codes, ones, sc, st)
    np.testing.assert_array_equal(w8, codes.astype(np.int64) - 8)
    np.testing.assert_array_equal(acc, a.astype(np.int64) @ (codes.astype(np.int64) - 8).T)
    want = (acc.astype(np.float32) * sc[None, :]) * st[:, None]            # (acc * s_ch) * s_tok
    np.testing.assert_array_equal(f, want)
    np.testing.assert_array_equal(q, np.clip(np.rint(want), -128, 127))


def test_w4a8_group_scale_rounds_the_exact_product_half_to_even():
    a = np.zeros((1, 128), np.int8)
    a[0, :16] = 1
    codes = np.arange(16, dtype=np.uint8)[None, :].repeat(1, 0)
    codes = np.pad(codes, ((0, 0), (0, 112)), constant_values=8)
    for s, want in [(0.5, [-4, -4, -3, -2, -2, -2, -1, 0, 0, 0, 1, 2, 2, 2, 3, 4]),      # x.5 ties go to even
                    (2.5, [-20, -18, -15, -12, -10, -8, -5, -2, 0, 2, 5, 8, 10, 12, 15, 18]),
                    (15.875, None)]:
        w8, acc, _, _ = oracle.gemm_w4a8(a, codes, np.full((1, 1), s, np.float16), np.float32([1]), np.float32([1]))
        exact = (np.arange(16) - 8) * float(np.float16(s))
        np.testing.assert_array_equal(w8[0, :16], np.rint(exact) if want is None else want)
        assert acc[0, 0] == w8[0, :16].astype(int).sum()
    # one scale per 128-code group and per column
    a, codes, sg, sc, st = _w4_case(4, 6, 384, 5)
    w8, _, _, _ = oracle.gemm_w4a8(a, codes, sg, sc, st)
    want = np.rint((codes.astype(np.float64) - 8) * np.repeat(sg.astype(np.float64), 128, axis=0).T)
    np.testing.assert_array_equal(w8, want)


def test_w4a8_per_channel_mode_shifts_the_signed_nibble():
    a, _, _, sc, st = _w4_case(5, 7, 128, 7)
    signed = np.random.default_rng(1).integers(-7, 8, (7, 128))
    w8, acc, _, _ = oracle.gemm_w4a8(a, (signed & 0xF).astype(np.uint8), None, sc, st)
    np.testing.assert_array_equal(w8, 16 * signed)
    np.testing.assert_array_equal(acc, a.astype(np.int64) @ (16 * signed).T)


def test_w4a8_quantiser_and_packing_round_trip():
    import torch
    from quamba_amd import w4a8_utils as wu
    g = torch.Generator().manual_seed(0)
    w = torch.randn(256, 96, generator=g) * 0.05                         # (K, N)
    w_ref, q_w, s_group, s_channel = wu.get_w4a8_quantize_weights(w, 4, 128)
    assert q_w.min() >= 0 and q_w.max() <= 15 and s_group.dtype == torch.float16 and s_group.shape == (2, 96)
    raw = w.reshape(2, 128, 96).abs().amax(1) * 2 / 15                   # group scale before the fusion
    deq = (q_w.reshape(2, 128, 96) - 8) * raw[:, None, :]
    assert (deq.reshape(256, 96) - w).abs().max() <= raw.max() * 0.5 + 1e-6    # half a step at most, except ...
    torch.testing.assert_close(s_group.float() * s_channel, raw, rtol=2e-3, atol=0)
    # the int8 second level reproduces w_ref: w8 * s_channel == w_ref
    w8 = torch.round((q_w.reshape(2, 128, 96) - 8) * s_group.float()[:, None, :]).reshape(256, 96)
    torch.testing.assert_close(w8 * s_channel, w_ref.float(), rtol=1e-2, atol=float(s_channel.max()))
    packed = wu.pack_w4a8(q_w)
    assert packed.shape == (96, 128) and packed.dtype == torch.uint8
    assert torch.equal(wu.unpack_w4a8(packed), q_w)
    # byte layout: byte i of word w = code[8w+i] | code[8w+4+i] << 4
    col = q_w[:, 5]
    assert int(packed[5, 0]) == int(col[0]) | (int(col[4]) << 4)
    assert int(packed[5, 7]) == int(col[11]) | (int(col[15]) << 4)
    # per-channel mode: signed 4-bit codes, channel scale pre-divided by 16
    w_ref2, q2, sg2, sc2 = wu.get_w4a8_quantize_weights(w[:128], 4, -1)
    assert q2.min() >= -7 and q2.max() <= 7 and sg2.numel() == 0
    torch.testing.assert_close((16 * q2) * sc2, w_ref2.float(), rtol=1e-3, atol=1e-6)
