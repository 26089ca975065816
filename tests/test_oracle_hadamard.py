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


def test_dense_stage_is_exact_whatever_the_order():
    """The dense B stage of the non-power-of-two rotations works on integers of at most 18 bits, so its sums are exact: Python-int
    arithmetic in shuffled orders gives the oracle's value, and fp32 accumulation in any order cannot round."""
    import random

    rng = np.random.default_rng(5)
    for n in (1408, 224):                                                  # 176 x 8 (S_4 kron B_44) and 28 x 8
        x = (rng.standard_normal((3, n)) * rng.choice([1e-3, 1.0, 300.0])).astype(F16)
        hk, k = O.get_hadK(n)
        m = n // k
        f, kb, b = O.had_factor(k)
        v = (O.sylvester_fwht(x.astype(np.float32).reshape(-1, k, m)) * O.had_scale(n)).astype(np.float32).astype(F16)
        to_grid, from_grid = O.dense_grid(v.reshape(3, n))
        for r in range(3):
            tg, fg = float(to_grid[r, 0]), float(from_grid[r, 0])
            mx = float(np.abs(v[r]).max())
            assert tg == 2.0 ** round(np.log2(tg)) and tg * fg == 16.0      # powers of two, from_grid = 16 / to_grid
            assert 2.0**16 <= mx * tg < 2.0**17                             # the largest value lands in [2^16, 2^17)
            q = [[int(np.rint(np.float32(v[r, kk, j]) * np.float32(tg))) for j in range(m)] for kk in range(k)]
            assert max(abs(e) for row in q for e in row) <= 2**17
            # snapping moves nothing by more than half a grid step
            assert max(abs(q[kk][j] / tg - float(v[r, kk, j])) for kk in range(k) for j in range(m)) <= 0.5 / tg
            y = O.online_hadamard(x[r:r + 1]).reshape(k, m)
            order = list(range(kb))
            for trial in range(3):
                random.Random(trial).shuffle(order)
                # integer sums in a shuffled order, then the S_f butterflies and the single rounding as defined
                t = np.zeros((f, kb, m), np.float32)
                for blk in range(f):
                    for bb in range(kb):
                        for j in range(m):
                            tot = 0
                            for bp in order:
                                tot += int(b[bb, bp]) * q[blk * kb + bp][j]
                                assert abs(tot) < 2**24                     # every partial sum is exact in fp32
                            t[blk, bb, j] = np.float32(tot) * np.float32(fg) / np.float32(16.0)
                t = np.moveaxis(O.sylvester_fwht(np.ascontiguousarray(np.moveaxis(t, 0, -1))), -1, 0)
                assert np.array_equal(t.astype(F16).reshape(k, m).view(np.uint16), y.view(np.uint16))


def test_dense_stage_on_grid_inputs_equals_the_plain_sum():
    """Rows whose values already sit on the grid (small integers) are not moved: the rotation is then the exact integer transform."""
    n = 224
    hk, k = O.get_hadK(n)
    rng = np.random.default_rng(6)
    x = rng.integers(-3, 4, size=(2, n)).astype(F16)
    dense = np.kron(hk.astype(np.float64), hadamard(n // k).astype(np.float64))
    want = ((x.astype(np.float64) @ dense.T).astype(np.float32) * O.had_scale(n)).astype(np.float32)
    y = O.online_hadamard(x)
    # step 1 rounds H_8 x / sqrt(224) to fp16 before the dense stage, so agreement is to fp16 rounding of those 28 terms ...
    assert np.abs(y.astype(np.float64) - want).max() <= 28 * 2.0**-11 * np.abs(want).max()
    # ... and exact when that rounding is exact: a row with one non-zero entry gives +-x/sqrt(n) everywhere
    e = np.zeros((1, n), F16)
    e[0, 37] = 5.0
    ye = O.online_hadamard(e)
    assert np.array_equal(np.abs(ye), np.full((1, n), np.float16(np.float32(5.0) * O.had_scale(n)), F16))
    assert np.array_equal(np.sign(ye[0]).astype(np.int64), dense[:, 37].astype(np.int64))


def test_dense_grid_edge_rows():
    z = np.zeros((1, 16), F16)
    assert O.dense_grid(z)[0][0, 0] == 1.0 and O.dense_grid(z)[1][0, 0] == 1.0
    tiny = np.full((1, 16), 2.0**-24, F16)                                   # the smallest fp16 subnormal: E = -23
    tg, fg = O.dense_grid(tiny)
    assert tg[0, 0] == 2.0**40 and fg[0, 0] == 2.0**-36
    big = np.full((1, 16), 65504.0, F16)
    tg, fg = O.dense_grid(big)
    assert tg[0, 0] == 2.0 and fg[0, 0] == 8.0
