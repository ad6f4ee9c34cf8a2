"""Pins the CPU oracle's Hadamard + quantisation restatement (no GPU): the fixed 12- and 40-point matrices
are Hadamard matrices with the reference's normalisation, the full transform equals the dense Kronecker
product in float64, it is an involution up to dim, and unit vectors pick out matrix columns exactly."""
import numpy as np
import pytest
import scipy.linalg

import oracle


@pytest.mark.parametrize("S", [12, 40])
def test_special_matrices_are_hadamard_with_the_reference_normalisation(S):
    H = oracle.hadamard_special(S).astype(int)
    np.testing.assert_array_equal(H @ H.T, S * np.eye(S, dtype=int))
    if S == 40:
        assert np.all(H[:, 0] == 1)
        # first row of the 20 x 20 core block: + followed by nineteen -; lower right block negated
        np.testing.assert_array_equal(H[0, :20], [1] + [-1] * 19)
        np.testing.assert_array_equal(H[:20, :20], -H[20:, 20:])
        np.testing.assert_array_equal(H[:20, :20], H[20:, :20])
        # circulant core: every row is the previous one rotated right by one
        core = H[1:20, 1:20]
        for i in range(1, 19):
            np.testing.assert_array_equal(core[i], np.roll(core[i - 1], 1))
    else:
        # rows 0 and 1 of Paley's second construction for q = 5
        np.testing.assert_array_equal(H[0], [1, -1] + [1] * 10)
        np.testing.assert_array_equal(H[1], [-1, -1] + [1, -1] * 5)
        np.testing.assert_array_equal(H, H.T)                      # the construction is symmetric


@pytest.mark.parametrize("S,name", [(12, "had_12_paley"), (40, "had_40_tpal")])
def test_special_matrices_equal_the_tables_the_reference_generates_its_code_from(S, name):
    # tests/golden/hadamard_tables.npz holds the +/- tables of the reference's csrc/hadamard/code_gen.py, parsed
    # as text by tests/golden/make_hadamard_tables.py; H H^T = n I alone would admit any Hadamard matrix
    import os
    tables = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hadamard_tables.npz"))
    np.testing.assert_array_equal(oracle.hadamard_special(S), tables[name])


def _dense(dim):
    S, M = oracle.hadamard_split(dim)
    W = scipy.linalg.hadamard(M).astype(np.float64) if M > 1 else np.ones((1, 1))
    Hs = oracle.hadamard_special(S).astype(np.float64) if S > 1 else np.ones((1, 1))
    return np.kron(Hs, W)


@pytest.mark.parametrize("dim", [8, 64, 96, 160, 1536, 5120, 2048])
def test_matches_dense_kronecker_product(dim):
    g = np.random.default_rng(dim)
    x = g.integers(-3, 4, (5, dim)).astype(np.float16)          # small integers: every fp32 sum is exact
    scale = np.float32(7.3 / np.sqrt(dim))
    want_f = (x.astype(np.float64) @ _dense(dim).T) * np.float64(scale)
    got = oracle.hadamard_quant(x, scale)
    # exact sums, so only the final fp32 product rounding separates the two: identical away from ties
    want = np.clip(np.where(want_f >= 0, np.floor(want_f + 0.5), np.ceil(want_f - 0.5)), -128, 127)
    tie = np.abs(np.abs(want_f - np.trunc(want_f)) - 0.5) < 1e-4
    np.testing.assert_array_equal(got[~tie], want[~tie].astype(np.int8))
    assert got.std() > 3


@pytest.mark.parametrize("dim", [32, 96, 640])
def test_unit_vectors_select_columns(dim):
    H = _dense(dim)
    x = np.eye(dim, dtype=np.float16) * np.float16(5.0)
    got = oracle.hadamard_quant(x, 1.0)
    np.testing.assert_array_equal(got, (5 * H.T).astype(np.int8))


def test_saturation_and_half_away_rounding():
    x = np.zeros((1, 8), np.float16)
    x[0, 0] = 1.0
    np.testing.assert_array_equal(oracle.hadamard_quant(x, 2.5)[0], [3] * 8)         # 2.5 rounds away from zero
    np.testing.assert_array_equal(oracle.hadamard_quant(-x, 2.5)[0], [-3] * 8)
    np.testing.assert_array_equal(oracle.hadamard_quant(x, 1000.0)[0], [127] * 8)
    np.testing.assert_array_equal(oracle.hadamard_quant(-x, 1000.0)[0], [-128] * 8)


def test_real_valued_rows_within_one_step_of_float64():
    dim = 5120
    g = np.random.default_rng(1)
    x = (g.standard_normal((4, dim)) * 3).astype(np.float16)
    scale = np.float32(1.0 / np.sqrt(dim) / 0.05)
    want = (x.astype(np.float64) @ _dense(dim).T) * np.float64(scale)
    got = oracle.hadamard_quant(x, scale).astype(np.float64)
    assert np.max(np.abs(got - np.clip(want, -128, 127))) <= 0.5 + 1e-3
