"""Pins oracle.quant_minmax / dequant / epilogue / int_gemm / silu_mul by known answers, closed forms and brute force."""
import numpy as np
import pytest

from oracle import mxmoe_oracle as O

F16 = np.float16


def test_sym_int4_known_answers_with_ties():
    # absmax 7 -> scale exactly 1; x/scale ties go to even AFTER the clamp (quant.py:82).
    x = np.array([[7, 0.5, 1.5, 2.5, 6.5, -0.5, -1.5, -2.5, -6.5, 3.49, -7, 100 * 0]], dtype=F16)
    q, s, z = O.quant_minmax(x, 4, -1, True)
    assert s.item() == 1.0 and z.item() == 0
    assert q.tolist() == [[7, 0, 2, 2, 6, -0, -2, -2, -6, 3, -7, 0]]


def test_sym_int8_known_answers():
    x = np.array([[127, -127, 63.5, 64.5, 1, -1]], dtype=F16)
    q, s, _ = O.quant_minmax(x, 8, -1, True)
    assert s.item() == 1.0
    assert q.tolist() == [[127, -127, 64, 64, 1, -1]]
    # a scale that is not a power of two: absmax 2 -> scale = fp16(2/127)
    x = np.array([[2.0, 1.0, -0.25]], dtype=F16)
    q, s, _ = O.quant_minmax(x, 8, -1, True)
    sc = F16(F16(2.0) / F16(127))
    assert s.item() == sc
    exp = [np.rint(np.clip(F16(v / sc), -127, 127)) for v in x[0]]
    assert q[0].tolist() == exp and q[0, 0] == 127


def test_clamp_happens_before_round():
    # x/scale = 7.5 would round to 8 if rounded first; clamp-then-round gives 7.
    x = np.array([[7.0, 7.5 * 0 + 7.0]], dtype=F16)
    q, _, _ = O.quant_minmax(x, 4, -1, True)
    assert q.max() == 7
    # asym: value above max cannot occur, but the closed form must still clamp to 2^b-1
    x = np.array([[0.0, 15.0, 7.5, 8.5]], dtype=F16)
    q, s, z = O.quant_minmax(x, 4, -1, False)
    assert s.item() == 1.0 and z.item() == 0.0
    assert q.tolist() == [[0, 15, 8, 8]]


def test_asym_group_known_answers():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((6, 256)).astype(F16)
    for bits in (4, 3):
        q, s, z = O.quant_minmax(x, bits, 128, False)
        g = x.reshape(-1, 128)
        qg = q.reshape(-1, 128)
        up = (1 << bits) - 1
        assert s.shape == (12, 1) and z.shape == (12, 1)
        assert np.array_equal(z[:, 0], g.min(axis=1))                      # float zero-point = group min
        assert np.array_equal(s[:, 0], ((g.max(1) - g.min(1)).astype(F16) / F16(up)).astype(F16))
        assert qg.min() >= 0 and qg.max() <= up
        assert np.all(qg[np.arange(12), g.argmin(1)] == 0)                 # min -> 0
        assert np.all(qg[np.arange(12), g.argmax(1)] >= up - 1)            # max -> 2^b-1 (up to fp16 rounding of the ratio)
        deq = O.dequant(q, s, z, 128)
        err = np.abs(deq.astype(np.float64) - x.astype(np.float64)).reshape(-1, 128)
        assert np.all(err <= s.astype(np.float64) * 0.5 * 1.01 + 2e-3)


def test_zero_group_guard_and_reference_nan():
    x = np.zeros((2, 8), dtype=F16)
    q, s, _ = O.quant_minmax(x, 4, -1, True)                               # quantize.cuh:258 guard
    assert np.all(s == 1) and np.all(q == 0)
    q, s, _ = O.quant_minmax(x, 4, -1, True, zero_guard=False)             # quant.py: 0/0 -> NaN
    assert np.all(np.isnan(q))


@pytest.mark.parametrize("bits", [4, 8])
def test_sym_sweep_all_fp16_against_float64_closed_form(bits):
    # every finite fp16 value v paired with an absmax element A, one row each: q(v) must equal
    # RNE(clamp(fp16(v / fp16(A/upper)))) evaluated independently in float64 with explicit fp16 roundings.
    allv = np.arange(0, 1 << 16, dtype=np.uint16).view(F16)
    allv = allv[np.isfinite(allv)]
    up = (1 << (bits - 1)) - 1
    for A in (F16(1.0), F16(3.3), F16(0.0117), F16(1000.0)):
        v = allv[np.abs(allv) <= A]
        rows = np.stack([v, np.full_like(v, A)], axis=1)
        q, s, _ = O.quant_minmax(rows, bits, -1, True)
        sc = np.float64(F16(np.float64(A) / up))                           # one fp16 rounding
        assert np.all(s[:, 0] == F16(sc))
        ratio = (v.astype(np.float64) / sc).astype(F16).astype(np.float64) # one fp16 rounding (exact quotient -> fp16)
        exp = np.rint(np.clip(ratio, -up, up))
        assert np.array_equal(q[:, 0].astype(np.float64), exp)
        assert np.all(q[:, 1] == up)                                       # absmax element -> +upper
        assert np.all(np.abs(q) <= up)


def test_int_gemm_matches_python_int_bruteforce():
    rng = np.random.default_rng(1)
    a = rng.integers(-127, 128, size=(5, 37))
    b = rng.integers(-127, 128, size=(7, 37))
    acc = O.int_gemm(a, b)
    for m in range(5):
        for n in range(7):
            assert int(acc[m, n]) == sum(int(a[m, k]) * int(b[n, k]) for k in range(37))
    assert acc.dtype == np.int32 and acc.shape == (5, 7)                   # [M, N], not transposed
    # worst-case magnitude at the largest K of the benchmark workloads (14336) stays inside int32
    k = 14336
    assert O.int_gemm(np.full((1, k), 127), np.full((1, k), -127))[0, 0] == -127 * 127 * k


def test_epilogue_closed_forms():
    acc = np.array([[3, -70000], [2**24 + 1, 5]], dtype=np.int32)
    one = np.ones(2, dtype=F16)
    out = O.epilogue_wxax(acc, one, one)                                   # sa=sb=1: int -> fp32 -> fp16 conversion
    assert out[0, 0] == 3 and np.isinf(out[0, 1]) and out[1, 1] == 5
    sa = np.array([0.1, 0.013], dtype=F16)
    sb = np.array([0.02, 0.5], dtype=F16)
    out = O.epilogue_wxax(acc, sa, sb)
    lit = O.epilogue_wxax(acc, sa, sb, scale_product="fp16")
    for m in range(2):
        for n in range(2):
            s32 = np.float32(sa[m]) * np.float32(sb[n])                    # exact in fp32 (11 + 11 significant bits)
            assert float(s32) == float(sa[m]) * float(sb[n])
            assert out[m, n] == F16(np.float32(acc[m, n]) * s32)
            s16 = F16(sa[m] * sb[n])                                       # the reference kernel rounds the product to fp16 first
            assert lit[m, n] == F16(np.float32(acc[m, n]) * np.float32(s16))
    # sa indexes rows (tokens), sb columns (channels): swapping them must change the result
    assert not np.array_equal(out, O.epilogue_wxax(acc, sb, sa))
    # typical int8 scales: the fp16 product is subnormal and off by percents, the fp32 product is not
    sa8, sb8 = np.array([0.001], dtype=F16), np.array([0.0007], dtype=F16)
    exact = 1000 * float(sa8[0]) * float(sb8[0])
    a1000 = np.array([[1000]], dtype=np.int32)
    assert abs(float(O.epilogue_wxax(a1000, sa8, sb8)[0, 0]) / exact - 1) < 1e-3
    assert abs(float(O.epilogue_wxax(a1000, sa8, sb8, "fp16")[0, 0]) / exact - 1) > 5e-3


def test_fakequant_path_agrees_with_integer_path_within_tolerance():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((33, 256)).astype(F16)
    w = (rng.standard_normal((48, 256)) * 0.02).astype(F16)
    for qp in [(4, 4, -1, True), (8, 8, -1, True)]:
        ok, of, acc = O.linear_block(x, w, qp, rotate=True)
        rel = np.abs(ok.astype(np.float64) - of.astype(np.float64)).max() / np.abs(of.astype(np.float64)).max()
        assert rel < 1e-2 and acc.dtype == np.int32


def test_fma_f32_is_one_correct_rounding():
    """The oracle's fused multiply-add against exact rational arithmetic, including products that cancel against the addend and
    results that sit next to a float32 rounding boundary (where rounding the float64 sum a second time would go wrong)."""
    from fractions import Fraction

    rng = np.random.default_rng(8)
    n = 3000
    a = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 6, n)).astype(np.float32)
    b = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 6, n)).astype(np.float32)
    c = (rng.standard_normal(n) * 10.0 ** rng.integers(-8, 8, n)).astype(np.float32)
    c[:1000] = (-(a[:1000].astype(np.float64) * b[:1000].astype(np.float64))).astype(np.float32)          # near-total cancellation
    # a * b = (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24; with c = 2^-24 + tiny the exact sum lies just above a float32 tie
    a[1000:1010] = np.float32(1 + 2.0**-12)
    b[1000:1010] = np.float32(1 + 2.0**-12)
    c[1000:1010] = np.float32(2.0**-24) * np.float32(1 + 2.0**-20) * np.arange(1, 11, dtype=np.float32)
    got = O.fma_f32(a, b, c)

    def exact(x, y, z):
        v = Fraction(float(x)) * Fraction(float(y)) + Fraction(float(z))
        near = np.float32(float(v))
        best = None
        for cand in (near, np.nextafter(near, np.float32(np.inf)), np.nextafter(near, np.float32(-np.inf))):
            key = (abs(Fraction(float(cand)) - v), int(np.asarray(cand).view(np.uint32)) & 1)   # nearest, ties to even
            if best is None or key < best[0]:
                best = (key, cand)
        return best[1]

    for i in range(n):
        assert got[i] == exact(a[i], b[i], c[i]), i
    assert O.fma_f32(np.float32(3), np.float32(4), np.float32(5)) == 17


def test_exp_fixed_and_silu_mul():
    """The two fixed sequences behind SiLU against float64 (relative error bounds that a wrong coefficient, a dropped Newton step or a
    wrong seed would break), and silu(g) * u against the float64 value for EVERY finite fp16 gate and several up values: within one
    fp16 ulp (0.52 at worst; a correctly rounded result would be within 0.5)."""
    gg = np.linspace(-69, 69, 100001).astype(np.float32)
    rel = np.abs(O.exp2_neg_f32_fixed(gg).astype(np.float64) / np.exp(-gg.astype(np.float64)) - 1)
    assert rel.max() < 1e-5
    assert O.exp2_neg_f32_fixed(np.float32(0.0)) == np.float32(1.0000001)          # k = 0, f = 0: the polynomial's constant term
    big = O.exp2_neg_f32_fixed(np.array([-1e4, 1e4, np.inf, -np.inf], np.float32))       # clamped at 2^+-100: finite, normal, no overflow
    assert np.all(np.isfinite(big)) and big[0] > 1e30 and 0 < big[1] < 1e-30 and big[0] == big[3] and big[1] == big[2]
    d = np.exp2(np.linspace(0, 101, 100001)).astype(np.float32)
    assert np.abs(O.rcp_f32_fixed(d).astype(np.float64) * d - 1).max() < 8e-6
    seed_only = (np.int32(0x7EF31000) - d.view(np.int32)).view(np.float32)
    assert 0.04 < np.abs(seed_only.astype(np.float64) * d - 1).max() < 0.051               # the seed alone is a 5 % guess: the Newton steps do the work
    g = np.arange(65536, dtype=np.uint16).view(F16)
    g = g[np.isfinite(g)]
    worst = 0.0
    for uval in (1.0, 0.333, -2.5, 1000.0, 6e-5):
        u = np.full_like(g, F16(uval))
        y = O.silu_mul(np.concatenate([g[None], u[None]], axis=1))[0]
        g64, u64 = g.astype(np.float64), u.astype(np.float64)
        with np.errstate(over="ignore"):
            ref = g64 / (1 + np.exp(-g64)) * u64
        fin = np.abs(ref) < 65504
        ulp = np.maximum(2.0 ** np.floor(np.log2(np.maximum(np.abs(ref), 1e-30))) * 2.0 ** -10, 2.0 ** -24)
        err = np.abs(y.astype(np.float64) - ref)[fin] / ulp[fin]
        worst = max(worst, err.max())
        assert np.all(np.isinf(y[~fin]) | (np.abs(y[~fin].astype(np.float64)) >= 65504 * (1 - 2.0 ** -11)))
    assert worst < 0.53
    rng = np.random.default_rng(3)
    gu = (rng.standard_normal((17, 64)) * 3).astype(F16)
    gu[0, :4] = [F16(-60000), F16(60000), F16(0), F16(-0.0)]
    y = O.silu_mul(gu)
    assert y.shape == (17, 32) and y[0, 0] == 0 and y[0, 2] == 0
    # first half is the gate: swapping halves changes the answer
    assert not np.array_equal(y, O.silu_mul(np.concatenate([gu[:, 32:], gu[:, :32]], axis=1)))


def test_grouped_accumulators_and_epilogue():
    rng = np.random.default_rng(21)
    m, n, k, g = 5, 7, 384, 128
    qa = rng.integers(-7, 8, (m, k)).astype(np.float16)
    qb = rng.integers(-7, 8, (n, k)).astype(np.float16)
    acc = O.int_gemm_grouped(qa, qb, g)
    assert acc.shape == (3, m, n)
    assert np.array_equal(acc.sum(axis=0), O.int_gemm(qa, qb))                       # the groups partition K
    assert np.array_equal(acc[1], O.int_gemm(qa[:, 128:256], qb[:, 128:256]))
    ones_a, ones_b = np.ones((m, 3), np.float16), np.ones((n, 3), np.float16)
    h, f = O.epilogue_grouped(acc, ones_a, ones_b)
    assert np.array_equal(f, O.int_gemm(qa, qb).astype(np.float32))                  # unit scales: the exact integer product
    sa = rng.uniform(0.01, 0.2, (m, 3)).astype(np.float16)
    sb = rng.uniform(0.001, 0.02, (n, 3)).astype(np.float16)
    h1, _ = O.epilogue_grouped(acc[:1], sa[:, :1], sb[:, :1])                        # one group: the per-token / per-channel epilogue
    assert np.array_equal(h1.view(np.uint16), O.epilogue_wxax(acc[0], sa[:, 0], sb[:, 0]).view(np.uint16))
    h, f = O.epilogue_grouped(acc, sa, sb)
    exact = sum(acc[i].astype(np.float64) * sa[:, i].astype(np.float64)[:, None] * sb[:, i].astype(np.float64)[None, :] for i in range(3))
    assert np.abs(f - exact).max() <= 4 * 2.0 ** -24 * np.abs(exact).max() + 1e-12
    # a sign error or a transposed scale fails: swap sa's groups
    h_bad, _ = O.epilogue_grouped(acc, sa[:, ::-1].copy(), sb)
    assert not np.array_equal(h_bad, h)


def test_linear_block_group_format_agrees_with_fake_quant():
    rng = np.random.default_rng(22)
    x = rng.standard_normal((6, 256)).astype(np.float16)
    w = (rng.standard_normal((16, 256)) * 0.02).astype(np.float16)
    out_k, out_f, acc = O.linear_block(x, w, (4, 4, 128, True), rotate=True)
    assert acc.shape == (2, 6, 16)
    rel = np.abs(out_k.astype(np.float64) - out_f.astype(np.float64)).max() / np.abs(out_f.astype(np.float64)).max()
    assert rel <= 1e-2


# ---- the quantiser kernels divide a row by its scale with one shared reciprocal: exactness of that scheme ----
def _rne_shift(x, sh):
    """round-to-nearest-even of x / 2^sh for non-negative int64 arrays (sh array or scalar >= 1)"""
    sh = np.asarray(sh, dtype=np.int64)
    half = np.int64(1) << (sh - 1)
    q = x >> sh
    r = x & ((np.int64(1) << sh) - 1)
    up = (r > half) | ((r == half) & ((q & 1) == 1))
    return q + up.astype(np.int64)


def _rn24(x):
    """(mantissa in [2^23, 2^24), exponent e) with value ~= m * 2^e of the positive int64 array x rounded to 24 significant bits"""
    nb = np.floor(np.log2(x.astype(np.float64))).astype(np.int64) + 1          # bit length (exact for < 2^53; values here are)
    # fix possible off-by-one of the float log
    nb = np.where((np.int64(1) << (nb - 1)) > x, nb - 1, nb)
    nb = np.where((np.int64(1) << nb) <= x, nb + 1, nb)
    sh = nb - 24
    m = np.where(sh > 0, _rne_shift(x, np.maximum(sh, 1)), x << np.maximum(-sh, 0))
    e = sh.copy()
    over = m == (1 << 24)
    m = np.where(over, m >> 1, m); e = np.where(over, e + 1, e)
    return m, e


def test_shared_reciprocal_division_is_exact_for_all_fp16_pairs():
    """v / s as the kernels compute it (r = RN(1 / s) once per row; q0 = RN(v * r); e = v - s * q0 exactly, one fused operation;
    q = RN(q0 + e * r), one fused operation) against the correctly rounded quotient, in exact integer arithmetic, for every pair of
    11-bit mantissas: fp16 values are such mantissas times powers of two (subnormals have trailing zeros), signs are symmetric and
    no intermediate leaves the normal fp32 range, so this covers every finite fp16 pair.  Without the correction step the rounded
    product alone is wrong for a large share of the pairs, so the check can fail."""
    a, b = np.meshgrid(np.arange(1024, 2048, dtype=np.int64), np.arange(1024, 2048, dtype=np.int64), indexing="ij")
    a = a.ravel(); b = b.ravel()
    # y = RN24(1/b): 2^34 / b lies in (2^23, 2^24]
    num = np.int64(1) << 34
    yq, yr = num // b, num % b
    Y = yq + ((2 * yr > b) | ((2 * yr == b) & (yq & 1 == 1))).astype(np.int64)       # value y = Y * 2^-34 (Y = 2^24 only for b = 1024)
    # q0 = RN24(a * y)
    P = a * Y                                                                       # value a*y = P * 2^-34
    m0, e0 = _rn24(P)                                                                # q0 = m0 * 2^(e0 - 34)
    # e = a - b*q0 exactly, in units of 2^(e0-34)
    E = (a << (34 - e0)) - b * m0
    assert (np.abs(E) < (1 << 24)).all(), "remainder representable in fp32"
    # q1 = RN24(q0 + e*y): units of 2^(e0-34-34)
    S = (m0 << 34) + E * Y
    m1, e1 = _rn24(S)                                                                # q1 = m1 * 2^(e1 + e0 - 68)
    # true quotient RN24(a/b): a/b in (0.5, 2)
    big = a << 40
    tq, tr = big // b, big % b                                                      # a/b = (tq + tr/b) * 2^-40, tq < 2^41
    nb = np.where(tq >= (np.int64(1) << 40), 41, 40)
    sh = nb - 24
    mt = tq >> sh
    rem_hi = tq & ((np.int64(1) << sh) - 1)
    half = np.int64(1) << (sh - 1)
    gt = (rem_hi > half) | ((rem_hi == half) & (tr > 0))
    tie = (rem_hi == half) & (tr == 0)
    mt = mt + (gt | (tie & ((mt & 1) == 1))).astype(np.int64)
    et = sh - 40
    over = mt == (1 << 24); mt = np.where(over, mt >> 1, mt); et = np.where(over, et + 1, et)

    same = (m1 == mt) & ((e1 + e0 - 68) == et)
    assert same.all(), (a[~same][:5], b[~same][:5])
    plain = (m0 == mt) & ((e0 - 34) == et)
    assert 0.05 < (~plain).mean() < 0.6


def test_e4m3_codes_known_answers_and_round_trip():
    """fp8 (OCP e4m3): all 254 number codes decode and re-encode to themselves; hand-computed values and ties (to even) at the
    spacings of the normal range (1 + m/8), of the top binade (256 .. 448, spacing 32) and of the subnormals (multiples of 2^-9)."""
    from oracle import mxmoe_oracle as O

    codes = np.arange(256, dtype=np.uint8)
    vals = O.e4m3_decode(codes)
    num = ~np.isnan(vals)
    assert num.sum() == 254 and np.isnan(vals[0x7F]) and np.isnan(vals[0xFF])
    assert np.array_equal(O.e4m3_encode(vals[num]), codes[num])
    assert vals[0x7E] == 448.0 and vals[0xFE] == -448.0 and vals[0x38] == 1.0 and vals[0x01] == 2.0 ** -9 and vals[0x08] == 2.0 ** -6 and vals[0x3C] == 1.5
    # ties: halfway between 1.0 (mantissa 000, even) and 1.125 (001) -> 1.0; between 1.125 and 1.25 (010, even) -> 1.25
    assert list(O.e4m3_encode(np.array([1.0625, 1.1875, 1.0626, -1.1874]))) == [0x38, 0x3A, 0x39, 0xB9]
    # top binade: 416 (m 101) .. 448 (m 110, even): 432 -> 448; 400 is between 384 (100) and 416 (101) -> 384
    assert list(O.e4m3_encode(np.array([432.0, 400.0, 447.9, 240.0]))) == [0x7E, 0x7C, 0x7E, 0x77]
    # carry into the next binade: 1.97 -> 2.0; subnormals: 1.5 * 2^-9 -> 2 * 2^-9 (even), 0.5 * 2^-9 -> 0 (even), largest subnormal + half -> smallest normal
    assert list(O.e4m3_encode(np.array([1.97, 1.5 * 2.0 ** -9, 0.5 * 2.0 ** -9, 7.5 * 2.0 ** -9, 0.0, -0.0]))) == [0x40, 0x02, 0x00, 0x08, 0x00, 0x80]
    with pytest.raises(ValueError):
        O.e4m3_encode(np.array([449.0]))


def test_e4m3_against_an_independent_cast_and_the_quantiser_rule():
    """Every finite fp16 value up to 448 in magnitude: the oracle's codes equal a library cast to float8_e4m3fn (torch, used here as
    an independent implementation of the same standard format).  quant_e4m3: the row's largest magnitude lands on +-448, no code
    is NaN, a zero row has scale 1, and dequantised values are within half a spacing (2^-4 relative) of the scaled input."""
    import torch

    from oracle import mxmoe_oracle as O

    x = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    x = x[torch.isfinite(x) & (x.abs() <= 448)]
    want = x.float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(O.e4m3_encode(x.float().numpy()), want)
    rng = np.random.default_rng(3)
    t = (rng.standard_normal((64, 512)) * rng.uniform(1e-3, 30, (64, 1))).astype(F16)
    t[5] = 0
    c, s = O.quant_e4m3(t)
    v = O.e4m3_decode(c)
    assert not np.isnan(v).any() and s[5, 0] == 1 and (v[5] == 0).all()
    live = np.abs(t).max(axis=1) > 0
    assert np.all(np.abs(v[live]).max(axis=1) == 448.0)
    ratio = (t[live].astype(np.float64) / s[live].astype(np.float64))
    assert np.all(np.abs(v[live] - ratio) <= np.maximum(np.abs(ratio) * 2.0 ** -4, 2.0 ** -10) * 1.01 + np.abs(ratio) * 2.0 ** -10)
    # the torch mirror used to pack weights gives the same codes and scales
    from mxmoe_amd.quant import quant_e4m3

    tc, ts = quant_e4m3(torch.from_numpy(t))
    assert np.array_equal(tc.numpy(), c) and np.array_equal(ts.numpy().view(np.uint16), s.view(np.uint16))
    # and fp8_gemm on one-hot / unit operands returns the operand values themselves
    a = O.e4m3_encode(np.eye(8)[:, :8] * 1.0)
    assert np.array_equal(O.fp8_gemm(c[:3, :8], a), v[:3, :8])


def test_bf16_rounding_known_answers_and_an_independent_cast():
    """bfloat16 keeps 8 significant bits: 257 lies halfway between 256 and 258 and goes to the even 256, 259 to 260, 1 + 2^-8 to 1,
    1 + 3 * 2^-8 to 1 + 2^-6; values of the format are fixed points; a random sample agrees with torch's cast bit for bit."""
    import torch

    x = np.array([257.0, 259.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -257.0, 255.5, 3.0e38, 1.0e-40, 0.0, -0.0], dtype=np.float32)
    want = np.array([256.0, 260.0, 1.0, 1.0 + 2.0 ** -6, -256.0, 256.0, 3.0e38, 1.0e-40, 0.0, -0.0], dtype=np.float32)
    got = O.bf16_round(x)
    assert np.array_equal(got[:6], want[:6])
    assert np.array_equal(O.bf16_round(got), got)                           # idempotent
    assert np.array_equal(O.bf16_from_bits(O.bf16_bits(x)), got)
    rng = np.random.default_rng(5)
    r = np.concatenate([rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 200000).astype(np.float32), x])
    t = torch.from_numpy(r).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(O.bf16_round(r).view(np.uint32), t.view(np.uint32))
    a = O.bf16_round(rng.standard_normal((5, 64)).astype(np.float32))
    b = O.bf16_round(rng.standard_normal((7, 64)).astype(np.float32))
    ref = torch.from_numpy(a.astype(np.float64) @ b.astype(np.float64).T).to(torch.float32).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(O.gemm_bf16(a, b), ref)
