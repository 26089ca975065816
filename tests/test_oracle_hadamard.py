"""Pins the oracle's Hadamard pieces: textbook Sylvester matrix, table orthogonality, kron composition."""
import numpy as np
import pytest
from scipy.linalg import hadamard

from oracle import mxmoe_oracle as O

F16 = np.float16


@pytest.mark.parametrize("n", [2, 8, 64, 2048])
def test_fwht_is_the_sylvester_matrix(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((3, n))
    y = O.sylvester_fwht(x)
    assert np.allclose(y, x @ hadamard(n).T, rtol=0, atol=1e-9 * n)
    assert np.allclose(O.sylvester_fwht(y) / n, x, atol=1e-9 * n)           # involution
    e0 = np.zeros((1, n)); e0[0, 0] = 1
    assert np.array_equal(O.sylvester_fwht(e0), np.ones((1, n)))           # H e_0 = 1
    j = np.arange(n)
    e5 = np.zeros((1, n)); e5[0, 5 % n] = 1                                # H[i][j] = (-1)^popcount(i & j)
    sign = np.array([(-1) ** bin(i & (5 % n)).count("1") for i in j])
    assert np.array_equal(O.sylvester_fwht(e5)[0], sign)


@pytest.mark.parametrize("k", [12, 20, 28, 36, 40, 52, 60, 108, 140, 156, 172, 176])
def test_tables_are_hadamard(k):
    h = O.had_table(k).astype(np.int64)
    assert set(np.unique(h)) == {-1, 1}
    assert np.array_equal(h @ h.T, k * np.eye(k, dtype=np.int64))


def test_get_hadK_selection():
    assert O.get_hadK(2048)[1] == 1 and O.get_hadK(4096)[1] == 1
    assert O.get_hadK(1408)[1] == 176                                      # 1408 = 176 * 8
    assert O.get_hadK(14336)[1] == 28                                      # 14336 = 28 * 512
    assert O.get_hadK(5632)[1] == 176                                      # shared expert 4 * 1408


@pytest.mark.parametrize("n", [2048, 1408, 224, 14336])
def test_online_hadamard_equals_dense_kron(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((2, n)).astype(F16)
    hk, k = O.get_hadK(n)
    dense = np.kron(hk.astype(np.float64) if k > 1 else np.ones((1, 1)), hadamard(n // k).astype(np.float64)) / np.sqrt(n)
    ref = x.astype(np.float64) @ dense.T                                   # index p = k * (n/K) + j
    y = O.online_hadamard(x).astype(np.float64)
    assert np.abs(y - ref).max() <= 2.0**-10 * np.abs(ref).max() * 2 + 1e-6
    # norm preservation (orthogonal transform) within fp16 rounding
    assert np.allclose((y**2).sum(1), (x.astype(np.float64) ** 2).sum(1), rtol=3e-3)
    # the float64 restatement of the reference's pure-torch path is the same linear map
    assert np.allclose(O.matmul_hadU_f64(x), ref, atol=1e-9)


def test_had_scale_is_fp32_reciprocal_sqrt():
    assert O.had_scale(2048) == np.float32(1.0) / np.sqrt(np.float32(2048))
    assert O.had_scale(4096) == np.float32(1 / 64)


def test_had_factor_rebuilds_the_table():
    f, kb, b = O.had_factor(176)
    assert (f, kb) == (4, 44)
    assert np.array_equal(np.kron(hadamard(4), b.astype(np.int64)), O.had_table(176).astype(np.int64))
    f, kb, b = O.had_factor(28)
    assert (f, kb) == (1, 28) and np.array_equal(b, O.had_table(28))
