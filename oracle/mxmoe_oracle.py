"""CPU oracle for the mixed-precision MoE GroupGEMM path.  TEST INFRASTRUCTURE ONLY.

This module is a numpy restatement of the reference algorithm.  It is the checker for the HIP
path: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import it; nothing under ``mxmoe_amd/`` does, and the product never falls back to it.

Every function cites the reference lines it follows (paths relative to the reference root).

What pins each function (so that a dropped term, wrong sign, wrong index or transposed operand
fails a test in ``tests/test_oracle_*.py``):

* ``quant_minmax`` / ``dequant`` / ``fake_quant``  — hand-computed known answers incl. ties
  (round-half-even after clamp), a sweep over every finite fp16 value against a float64 closed
  form, invariants (|q| <= upper, absmax -> +-upper, group min -> 0, max -> 2^b-1).
* ``int_gemm``            — exact integer arithmetic vs a python-int brute force.
* ``epilogue_wxax``       — closed form incl. the sa = sb = 1 special case (int -> fp16 convert).
* ``int_gemm_grouped`` / ``epilogue_grouped`` — groups sum to ``int_gemm``; one group reduces to
  ``epilogue_wxax``; unit scales give the exact integer product; float64 sum within fp32 rounding.
* ``sylvester_fwht``      — scipy.linalg.hadamard dense product, involution, H e_0, Parseval.
* ``had_table``           — H H^T = K I and all entries +-1.
* ``online_hadamard``     — dense kron(H_K, H_{n/K}) / sqrt(n) in float64.
* ``had_factor``          — kron(S_f, B) rebuilt and compared with the table.
* ``route_topk``          — textbook softmax / top-k in float64, weights sum to one; hand-computed probabilities (logits = ln of
  small integers), equal logits in index order, torch.softmax + torch.topk as an independent library routine.
* ``permute_by_expert``   — brute force against a dict-of-lists.
* ``tile_to_problem``     — every (problem, tile_m, tile_n) visited exactly once.
* ``silu_mul`` / ``exp2_neg_f32_fixed`` / ``rcp_f32_fixed`` — float64 ``x*sigmoid(x)*u`` within one fp16 ulp for EVERY fp16 gate
  value; the two sequences against float64 exp and division (relative error bounds), exact-rational checks of ``fma_f32``.
* ``unpermute_combine``   — one-hot weights return the routed row bit for bit, dense float64 sum
  within fp16 rounding (+ shared row), independence of the order of the sorted rows, dropped slots.

Parity unpinned (see also the header of ``online_hadamard``): the reference's online rotation
calls the third-party ``fast_hadamard_transform`` CUDA package (Dao-AILab, version unpinned,
empty submodule in the reference) and an fp16 ``hadK @ x`` matmul whose accumulation order is
backend dependent.  None of the reference's files pins their last fp16 bit.  The order used here
is this build's own deterministic definition; agreement with the reference at that boundary is
"equal up to fp16 rounding of the rotated activation".  Also unpinned: the rounding inside
``silu_mul`` (the reference's kernel source for it, act_kernel.cuh, is absent; torch's fp16
``act_fn(g) * u`` rounds the activation to fp16 before the multiply, here silu(g) stays in fp32
and the product is rounded once; exp and the reciprocal are short fixed sequences accurate to 1e-5), at most one fp16 ulp of the
product apart.
* ``e4m3_encode`` / ``e4m3_decode`` / ``quant_e4m3`` / ``fp8_gemm`` — all 256 codes round-trip, hand-computed ties
  (to even) at normal, subnormal and top-of-range spacings, every fp16 value against an independent
  library cast (torch.float8_e4m3fn), absmax -> +-448; the fp8 format of the reference's w8a8_g-1_sym_E4M3 tiles
  has no quantiser in the reference (only the matrix instruction, mm_tile.cuh:696-697), so its scale rule
  (max / 448) is this build's definition: parity unpinned beyond "per-row scale, e4m3 codes, fp32 sums".
* ``bf16_round`` / ``bf16_bits`` / ``gemm_bf16`` — hand-computed ties (to even) on both sides of a binade, every float32 of a
  random sample against an independent library cast (torch.bfloat16), round trip through the bits.
* ``dense_grid`` / the exact dense stage of ``online_hadamard`` — python-int sums in shuffled
  orders give the same bits; grid edges (zero rows, subnormal and largest fp16 values).
* ``fma_f32`` — one correct rounding against exact rational arithmetic.
"""
from __future__ import annotations

from pathlib import Path

import numpy as np

F16 = np.float16
F32 = np.float32

_HAD_FILE = Path(__file__).resolve().parent.parent / "mxmoe_amd" / "data" / "had_tables.npz"


# --------------------------------------------------------------------------------------------
# Quantiser  (mxmoe/quant/quant.py:40-109; second statement mxmoe/kernels/src/include/quantize.cuh:218-279)
# --------------------------------------------------------------------------------------------
def quant_minmax(t: np.ndarray, bits: int, gsize: int, sym: bool, clip=(1.0, 1.0), zero_guard: bool = True):
    """Dynamic min/max quantisation along the last dim, in the dtype of ``t`` (fp16 in the path).

    Follows quant.py:61-84: groups are ``reshape(-1, gsize)``; sym: ``upper = 2^(b-1)-1``,
    ``scale = absmax / upper``, ``zp = 0``; asym: ``upper = 2^b-1``, ``scale = (max*c1 - min*c0) / upper``,
    ``zp = min*c0`` (a float zero point); ``q = round(clamp((x - zp) / scale, lower, upper))`` with
    clamp BEFORE the round-half-even.  Every operation rounds to ``t.dtype``.

    ``zero_guard`` follows quantize.cuh:258 (``scale == 0 -> 1``); quant.py has no guard and yields
    NaN for a constant-zero group.  Returns ``(q (t.shape, t.dtype), scale [G,1], zp [G,1])``.
    """
    dt = t.dtype
    g = t.shape[-1] if gsize == -1 else gsize
    r = t.reshape(-1, g)
    if sym:
        upper = float((1 << (bits - 1)) - 1)
        lower = -upper
        gmax = np.abs(r).max(axis=1, keepdims=True)
        scale = (gmax / dt.type(upper)).astype(dt)
        zp = np.zeros_like(scale)
    else:
        upper = float((1 << bits) - 1)
        lower = 0.0
        gmin = (r.min(axis=1, keepdims=True) * dt.type(clip[0])).astype(dt)
        gmax = (r.max(axis=1, keepdims=True) * dt.type(clip[1])).astype(dt)
        scale = ((gmax - gmin).astype(dt) / dt.type(upper)).astype(dt)
        zp = gmin
    if zero_guard:
        scale = np.where(scale == 0, dt.type(1), scale).astype(dt)
    with np.errstate(divide="ignore", invalid="ignore"):
        x = (r - zp).astype(dt)
        x = (x / scale).astype(dt)
    x = np.clip(x, dt.type(lower), dt.type(upper))
    q = np.rint(x).astype(dt)  # numpy rint == torch.round == round-half-to-even
    return q.reshape(t.shape), scale, zp


def dequant(q: np.ndarray, scale: np.ndarray, zp: np.ndarray, gsize: int) -> np.ndarray:
    """quant.py:99-102: ``q.reshape(-1, g) * scale + zp`` — two roundings in ``q.dtype``."""
    dt = q.dtype
    g = q.shape[-1] if gsize == -1 else gsize
    r = q.reshape(-1, g)
    return ((r * scale).astype(dt) + zp).astype(dt).reshape(q.shape)


def fake_quant(t: np.ndarray, bits: int, gsize: int, sym: bool, clip=(1.0, 1.0)) -> np.ndarray:
    """quant.py:104-106 (``bits == 16`` passes through, quant.py:95,100,105)."""
    if bits >= 16:
        return t
    q, s, z = quant_minmax(t, bits, gsize, sym, clip)
    return dequant(q, s, z, gsize)


# --------------------------------------------------------------------------------------------
# GEMMs and epilogues
# --------------------------------------------------------------------------------------------
def int_gemm(qa: np.ndarray, qb: np.ndarray) -> np.ndarray:
    """Integer accumulators of the w8a8 / w4a4 mainloop (cta_gemm.cuh:557-598): ``acc[m,n] = sum_k qa[m,k] qb[n,k]``.

    Computed exactly (float64 matmul of small integers is exact below 2^53) and returned as int32;
    asserts the int32 range the kernels accumulate in is not exceeded.
    """
    a = np.asarray(qa, dtype=np.float64)
    b = np.asarray(qb, dtype=np.float64)
    acc = a @ b.T
    assert np.abs(acc).max(initial=0) < 2**31
    return acc.astype(np.int64).astype(np.int32)


def epilogue_wxax(acc: np.ndarray, sa: np.ndarray, sb: np.ndarray, scale_product: str = "fp32") -> np.ndarray:
    """w-a epilogue (mm_tile.cuh:468-496 then :642-646): ``half(float(acc) * (sa[m] * sb[n]))``.

    ``sa`` [M] per-token and ``sb`` [N] per-channel fp16 scales.  The reference kernel rounds the scale product to
    fp16 (``T(r_sa * r_sb)`` on halves, mm_tile.cuh:490) before widening; for int8 scales that product is an fp16
    subnormal (~1e-6) and loses most of its mantissa, which alone exceeds the 1e-2 tolerance against the fake-quant
    path.  ``scale_product="fp32"`` (what the HIP kernels do) keeps the product of the two fp16 scales in fp32, where it
    is exact; ``"fp16"`` restates the reference kernel literally.  Then: fp32 multiply with the converted accumulator,
    one rounding to fp32, one to fp16.
    """
    a = sa.astype(F16).reshape(-1, 1)
    b = sb.astype(F16).reshape(1, -1)
    s = (a * b).astype(F16).astype(F32) if scale_product == "fp16" else (a.astype(F32) * b.astype(F32)).astype(F32)
    return (acc.astype(F32) * s).astype(F32).astype(F16)


def int_gemm_grouped(qa: np.ndarray, qb: np.ndarray, gsize: int) -> np.ndarray:
    """Integer accumulators of a group-quantised mainloop, one per K group: ``acc[g,m,n] = sum_{k in group g} qa[m,k] qb[n,k]``
    (cta_gemm.cuh:613-772 keeps one integer fragment per group before rescaling it)."""
    k = qa.shape[-1]
    assert k % gsize == 0
    return np.stack([int_gemm(qa[:, g * gsize:(g + 1) * gsize], qb[:, g * gsize:(g + 1) * gsize]) for g in range(k // gsize)])


def epilogue_grouped(acc: np.ndarray, sa: np.ndarray, sb: np.ndarray) -> np.ndarray:
    """Group-quantised w-a epilogue: ``half( sum_g float(acc[g]) * (sa[m,g] * sb[n,g]) )``.

    acc [G,M,N] int32, sa [M,G], sb [N,G] fp16.  Per group the product of the two fp16 scales is exact in fp32, the converted
    accumulator is multiplied by it (one fp32 rounding) and added to the running fp32 sum, groups in ascending order, starting from
    0 (one rounding per addition); one final rounding to fp16.  The reference rescales each group's integer fragment into an fp32
    fragment in the same ascending order (cta_gemm.cuh:613-772)."""
    g, m, n = acc.shape
    out = np.zeros((m, n), dtype=F32)
    for i in range(g):
        s = (sa[:, i].astype(F32).reshape(-1, 1) * sb[:, i].astype(F32).reshape(1, -1)).astype(F32)
        out = (out + (acc[i].astype(F32) * s).astype(F32)).astype(F32)
    return out.astype(F16), out


def gemm_fakequant(xq: np.ndarray, wq: np.ndarray) -> np.ndarray:
    """The fake-quant linear (quant.py:126-130 hook + ``F.linear``): ``xq @ wq.T`` on fp16 values.

    fp16 storage, float64 accumulation (the tightest reading of "what the mathematics fixes"),
    rounded once to fp16.  This is the value the 1e-2 max-abs-rel criterion compares against.
    """
    return (xq.astype(np.float64) @ wq.astype(np.float64).T).astype(F16)


def gemm_fp16(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """fp16 x fp16 -> fp32 accumulate -> fp16 (cta_gemm.cuh:8-107); float64 here, compared at 1e-2."""
    return gemm_fakequant(x, w)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32 values: the type of the reference's ``bf16`` tiles
    (tile_config.py:42, MMA_BF16_FP32: bf16 operands, fp32 accumulators, bf16 outputs).  numpy has no bfloat16, so the rounding is done
    on the bit pattern: add half of the dropped 16 bits' unit, plus the kept part's lowest bit minus one for the tie."""
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(F32)
    return np.where(np.isnan(x), F32(np.nan), out).astype(F32)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """The 16-bit storage of ``bf16_round(x)`` (upper half of the float32 pattern)."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(F32)


def gemm_bf16(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """bf16 x bf16 -> fp32 accumulate -> bf16 (cta_gemm.cuh:8-107 with the bf16 matrix instruction): ``x``, ``w`` hold bf16 values as
    float32; float64 sum, rounded to float32 and then to bf16 (compared at 1e-2, like the fp16 GEMM: the hardware's order of additions
    is its own)."""
    return bf16_round((x.astype(np.float64) @ w.astype(np.float64).T).astype(F32))


# --------------------------------------------------------------------------------------------
# SiLU * up  (input of the down projection)
# --------------------------------------------------------------------------------------------
_NEG_LOG2E = F32(-1.4426950408889634)
# 2^f on [-0.5, 0.5], degree 4, relative error 3.7e-6 (least squares on Chebyshev nodes), lowest coefficient first
_EXP2_C = [F32(c) for c in (1.0000001, 0.693121, 0.24022107, 0.05592204, 0.00967604)]
_RCP_SEED = np.int32(0x7EF31000)          # bits(seed) = this - bits(d): within 5.06 % of 1 / d for every positive normal d


def fma_f32(a, b, c) -> np.ndarray:
    """Fused multiply-add on float32 values: ``a * b + c`` rounded ONCE to float32 (what the GPU's v_fma_f32 computes).

    The product of two float32 values is exact in float64; the sum is taken in float64 with its exact rounding error (TwoSum),
    and an inexact sum gets its last bit set (round to odd), after which the rounding to float32 cannot go wrong (53 >= 2*24 + 2).
    """
    a = np.asarray(a, F32).astype(np.float64)
    b = np.asarray(b, F32).astype(np.float64)
    c = np.asarray(c, F32).astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        p = a * b
        s = p + c
        bb = s - p
        err = (p - (s - bb)) + (c - bb)
        bits = s.view(np.int64)
        fix = (err != 0) & ((bits & 1) == 0) & np.isfinite(s)
        up = (err > 0) == (s > 0)
        bits = np.where(fix, np.where(up, bits + 1, bits - 1), bits)
        return bits.view(np.float64).astype(F32)


def exp2_neg_f32_fixed(g: np.ndarray) -> np.ndarray:
    """``exp(-g)`` in fp32 as a FIXED sequence of correctly rounded fp32 and exact integer operations, relative error < 1e-5:
    ``t = clamp(g * -log2(e), -100, 100)``, ``k = rint(t)``, ``f = t - k`` (exact), ``p = 2^f`` by a degree-4 Horner polynomial of
    fused multiply-adds, and ``2^k`` added to p's exponent field (p lies in [0.70, 1.42] and |k| <= 100, so the result stays a
    normal number).  The HIP kernels run the identical sequence."""
    g = np.asarray(g, F32)
    with np.errstate(invalid="ignore", over="ignore"):
        t = (g * _NEG_LOG2E).astype(F32)
        t = np.minimum(np.maximum(t, F32(-100.0)), F32(100.0))
        k = np.rint(t).astype(F32)
        f = (t - k).astype(F32)
        p = np.full_like(f, _EXP2_C[4])
        for c in _EXP2_C[3::-1]:
            p = fma_f32(p, f, c)
        return (p.view(np.int32) + (k.astype(np.int32) << 23)).view(F32)


def rcp_f32_fixed(d: np.ndarray) -> np.ndarray:
    """``1 / d`` for positive normal d as a fixed sequence: an integer-subtraction seed (within 5.06 %) refined by two Newton steps
    ``r <- fma(r, fma(-d, r, 1), r)``; relative error < 7e-6 (the fourth power of the seed's)."""
    d = np.asarray(d, F32)
    r = (_RCP_SEED - d.view(np.int32)).view(F32)
    for _ in range(2):
        r = fma_f32(r, fma_f32(-d, r, F32(1.0)), r)
    return r


def silu_mul(gate_up: np.ndarray) -> np.ndarray:
    """``silu(gate) * up`` on a fused ``[rows, 2I]`` fp16 tensor, first half = gate, second = up.

    Contract of the reference's ``silu_mul_then_quant_kernel`` launch (ref_bind.cu:691-716; kernel
    source absent from the reference).  fp32: ``s = g * rcp(1 + exp(-g))`` with the two fixed sequences above, ``y = s * u``, one
    fp16 rounding: within one fp16 ulp of the exact value (0.53 ulp at worst over every fp16 gate).
    """
    i = gate_up.shape[-1] // 2
    g = gate_up[..., :i].astype(F32)
    u = gate_up[..., i:].astype(F32)
    with np.errstate(invalid="ignore", over="ignore"):
        d = (F32(1.0) + exp2_neg_f32_fixed(g)).astype(F32)
        s = (g * rcp_f32_fixed(d)).astype(F32)
        return (s * u).astype(F32).astype(F16)


# --------------------------------------------------------------------------------------------
# Hadamard rotation  (mxmoe/quant/hadamard_utils.py:5-106, rotation.py:403-421)
# --------------------------------------------------------------------------------------------
_HAD_ORDER = (176, 172, 156, 140, 108, 60, 52, 36, 28, 40, 20, 12)  # hadamard_utils.py:7-56 test order


def had_table(k: int) -> np.ndarray:
    """K x K +-1 matrix (int8) — hadamard_utils.py:162-4379 tables, stored bit-packed."""
    z = np.load(_HAD_FILE)
    bits = np.unpackbits(z[f"had{k}"])[: k * k].reshape(k, k)
    return (1 - 2 * bits.astype(np.int8)).astype(np.int8)


def _is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


def get_hadK(n: int):
    """hadamard_utils.py:5-59: first K in the reference's test order with ``n % K == 0`` and ``n/K`` a power of two."""
    for k in _HAD_ORDER:
        if n % k == 0:
            assert _is_pow2(n // k)
            return had_table(k), k
    assert _is_pow2(n)
    return None, 1


def sylvester_fwht(x: np.ndarray) -> np.ndarray:
    """Unnormalised Walsh-Hadamard transform along the last dim (length 2^m), Sylvester order.

    Stages in ASCENDING stride h = 1, 2, 4, ...: ``(a, b) -> (a + b, a - b)`` for index pairs
    ``(i, i + h)`` with bit ``h`` of ``i`` clear.  Each op rounds in ``x.dtype``; with fp32 input
    every output is a fixed binary tree of fp32 adds, which the HIP kernel reproduces bit for bit.
    """
    n = x.shape[-1]
    assert _is_pow2(n)
    y = x.copy()
    h = 1
    while h < n:
        v = y.reshape(*y.shape[:-1], n // (2 * h), 2, h)
        a = v[..., 0, :].copy()
        b = v[..., 1, :].copy()
        v[..., 0, :] = a + b
        v[..., 1, :] = a - b
        h *= 2
    return y


def had_scale(n: int) -> np.float32:
    """``1.0 / torch.tensor(n).sqrt()`` (hadamard_utils.py:99,103): fp32 sqrt, fp32 reciprocal."""
    return F32(1.0) / np.sqrt(F32(n))


def had_factor(k: int):
    """Split ``H_K = S_f kron B`` with ``S_f`` the Sylvester matrix of the largest power of two ``f`` for which it holds.

    had176 of the reference's table is ``S_4 kron B_44``; had28 has no such factor (f = 1).  Returns ``(f, Kb, B int8)``.
    """
    h = had_table(k)
    f = 1
    while k % (2 * f) == 0:
        g = 2 * f
        b = k // g
        blk = h[:b, :b]
        ok = all(
            np.array_equal(h[i * b:(i + 1) * b, j * b:(j + 1) * b], ((-1) ** bin(i & j).count("1")) * blk)
            for i in range(g) for j in range(g)
        )
        if not ok:
            break
        f = g
    kb = k // f
    return f, kb, h[:kb, :kb].copy()


def dense_grid(v: np.ndarray):
    """Per-row power-of-two factors of the dense ``B`` stage of ``online_hadamard``: ``(to_grid, from_grid)`` float32 ``[rows, 1]``.

    With ``max|v| < 2^E`` over the row (E from the exponent field of the fp32 maximum; NaNs are ignored), ``to_grid = 2^(17-E)``
    maps the row onto integers of magnitude <= 2^17 and ``from_grid = 2^(E-13)`` maps sums of those integers divided by 16 (the
    form the HIP kernel feeds to the fp16 matrix instruction: at most 11 significant bits, 2^-4 <= |.| <= 2^13) back.  An
    all-zero row gets (1, 1).
    """
    mx = np.fmax.reduce(np.abs(v.astype(F32)), axis=1, keepdims=True).astype(F32)
    e_field = (mx.view(np.uint32) >> 23).astype(np.int64)
    to_grid = np.where(e_field == 0, 127 << 23, (270 - e_field) << 23).astype(np.uint32).view(F32)
    from_grid = np.where(e_field == 0, 127 << 23, np.maximum(e_field - 12, 1) << 23).astype(np.uint32).view(F32)
    return to_grid, from_grid


def online_hadamard(x: np.ndarray) -> np.ndarray:
    """Online rotation of fp16 rows: ``y = (H_K kron H_{n/K}) x / sqrt(n)``, index ``p = k*(n/K) + j``.

    Follows ``matmul_hadU_cuda`` (hadamard_utils.py:96-106): view ``[K, n/K]``, Sylvester transform
    of each length-``n/K`` row scaled by ``1/sqrt(n)`` and returned in fp16, then ``hadK @ .`` in fp16.
    PARITY UNPINNED at the last fp16 bit (third-party kernel + backend matmul order, see module
    header).  This build's definition, which the HIP kernels reproduce bit for bit:
      1. fp32 ``sylvester_fwht`` along ``n/K`` (ascending strides), one fp32 multiply by ``had_scale(n)``, round to fp16;
      2. K > 1, with ``H_K = S_f kron B`` (``had_factor``): the row's fp16 values are snapped (round to nearest even) to the
         grid of step ``2^(E-17)``, ``max|v| < 2^E`` over the row (``dense_grid``); inside each of the f blocks of Kb rows
         ``t[b] = sum_{b'} B[b,b'] v[b']`` is then an EXACT sum (integers below 2^17 times Kb <= 64 < 2^7 terms stay below
         2^24), so its value does not depend on the order or the width of the accumulation and the kernel may leave it to
         the matrix cores; then the ``S_f`` butterflies across blocks in fp32 (ascending strides); one rounding to fp16.
         Snapping moves a value by at most 2^-18 of the row's largest one, far below the fp16 rounding of step 1 and the
         int4 / int8 quantisation step that follows.  Rows that hold an infinity or a NaN give unspecified values.
    """
    assert x.dtype == F16
    n = x.shape[-1]
    hk, k = get_hadK(n)
    m = n // k
    v = x.astype(F32).reshape(-1, k, m)
    v = (sylvester_fwht(v) * had_scale(n)).astype(F32).astype(F16)
    if k == 1:
        return v.reshape(x.shape)
    f, kb, b = had_factor(k)
    assert kb <= 64
    rows = v.shape[0]
    to_grid, from_grid = dense_grid(v.reshape(rows, n))
    q = np.rint((v.astype(F32).reshape(rows, n) * to_grid).astype(F32)).reshape(rows, f, kb, m)  # integers, |q| <= 2^17
    with np.errstate(invalid="ignore", over="ignore"):
        t = np.einsum("cb,rfbm->rfcm", b.astype(np.float64), q.astype(np.float64) / 16.0)        # exact in float64
        acc = (t.astype(F32) * from_grid.reshape(rows, 1, 1, 1)).astype(F32)                     # exact: |16 t| < 2^24, power-of-two factor
    # S_f butterflies across the block index (axis 1): move it last, transform, move back
    acc = np.moveaxis(sylvester_fwht(np.ascontiguousarray(np.moveaxis(acc, 1, -1))), -1, 1)
    return acc.astype(F16).reshape(x.shape)


def matmul_hadU_f64(x: np.ndarray) -> np.ndarray:
    """float64 restatement of the pure-torch ``matmul_hadU`` (hadamard_utils.py:62-83), for cross-checks.

    Its butterfly pairs ADJACENT elements and concatenates sums then differences at every level
    (the ``view(.., n/2, 2, .)`` at :68-73), stopping at length K, then applies ``hadK @`` and ``/ sqrt(n)``.
    """
    n = x.shape[-1]
    hk, k = get_hadK(n)
    inp = x.astype(np.float64).reshape(-1, n, 1)
    while inp.shape[1] > k:
        b, l, w = inp.shape
        v = inp.reshape(b, l // 2, 2, w)
        inp = np.concatenate([v[:, :, 0, :] + v[:, :, 1, :], v[:, :, 0, :] - v[:, :, 1, :]], axis=-1)
    if k > 1:
        inp = hk.astype(np.float64)[None] @ inp
    return inp.reshape(x.shape) / np.sqrt(np.float64(n))


# --------------------------------------------------------------------------------------------
# Routing, permutation, offsets
# --------------------------------------------------------------------------------------------
def route_topk(logits: np.ndarray, topk: int, renormalise: bool = True):
    """moe_tracer.py:79-86: ``softmax(logits, fp32) -> topk -> (optionally) renormalise``.  Returns (ids int32 [T,k], weights fp32).

    Equal probabilities go to the lower expert id first (torch.topk leaves that order open).  ``renormalise`` divides the k weights
    by their sum (Mixtral's ``norm_topk_prob``); without it the weights are the plain probabilities (Qwen-MoE, DeepSeek-V2-Lite)."""
    z = logits.astype(F32)
    z = z - z.max(axis=1, keepdims=True)
    p = np.exp(z)
    p = p / p.sum(axis=1, keepdims=True)
    ids = np.argsort(-p, axis=1, kind="stable")[:, :topk]
    w = np.take_along_axis(p, ids, axis=1)
    if renormalise:
        w = w / w.sum(axis=1, keepdims=True)
    return ids.astype(np.int32), w.astype(F32)


def permute_by_expert(topk_ids: np.ndarray, num_experts: int):
    """ref_bind.cu:47-64,449-453: sort the flattened expert ids, ``perm = idx // topk``, ``bincount``.

    The reference's sort is unstable (order inside an expert unspecified); this build fixes the STABLE order.
    Returns ``(dst_exp_sorted int32 [R], perm_indices int64 [R] (source token of each sorted row),
    src_slot int64 [R] (flattened (token, slot) index), recv_tokens_per_exp int64 [E])``.
    """
    flat = topk_ids.reshape(-1).astype(np.int64)
    order = np.argsort(flat, kind="stable")
    k = topk_ids.shape[1]
    return flat[order].astype(np.int32), (order // k).astype(np.int64), order.astype(np.int64), np.bincount(flat, minlength=num_experts).astype(np.int64)


def act_tag(a_bits: int, gsize: int) -> int:
    """ref_bind.cu:461-473: 0 fp16, 1 int8 per-token, 2 int4 per-token, 3 int4 group-128, -1 unsupported."""
    if a_bits >= 16:
        return 0
    if a_bits == 8 and gsize == -1:
        return 1
    if a_bits == 4 and gsize == -1:
        return 2
    if a_bits == 4 and gsize == 128:
        return 3
    return -1


def act_offsets(recv: np.ndarray, num_tokens: int, qparams_per_exp, k_dim: int, has_shared: bool, shared_k_dim: int | None = None):
    """Per-expert exclusive offsets of the packed activation / scale stores (ref_bind.cu:475-505, 635-671).

    Units are fp16 elements, as in the reference: row strides ``K``, ``K/2``, ``K/4`` halves for tags
    0/1/2(3); scale strides 0 / 1 / 1 / ``K/128``.  The shared expert is index E with ``num_tokens`` rows.
    Returns dict of int64 arrays ``tag, start_row, inp_off, scale_off, inp_size, scale_size`` (length E(+1)).
    """
    e_tot = len(recv) + (1 if has_shared else 0)
    out = {k: np.zeros(e_tot, dtype=np.int64) for k in ("tag", "start_row", "inp_off", "scale_off", "inp_size", "scale_size")}
    rows = io = so = 0
    for e in range(e_tot):
        a_bits, _w, g, _s = qparams_per_exp[e]
        tag = act_tag(a_bits, g)
        kd = k_dim if (e < len(recv) or shared_k_dim is None) else shared_k_dim
        ld = kd if tag == 0 else (kd // 2 if tag == 1 else kd // 4)
        sld = 0 if tag == 0 else (1 if tag in (1, 2) else kd // 128)
        n = num_tokens if e == len(recv) else int(recv[e])
        out["tag"][e], out["start_row"][e], out["inp_off"][e], out["scale_off"][e] = tag, rows, io, so
        out["inp_size"][e], out["scale_size"][e] = ld * n, sld * n
        rows += n
        io += ld * n
        so += sld * n
    return out


# --------------------------------------------------------------------------------------------
# fp8 (OCP e4m3) — the operand format of the reference's w8a8_g-1_sym_E4M3 tiles (mxmoe/kernels/tile_config.py:45,192,
# mma.sync ... e4m3.e4m3.f32, mxmoe/kernels/src/include/cuda_utils.cuh:385-410)
# --------------------------------------------------------------------------------------------
E4M3_MAX = 448.0


def e4m3_decode(code: np.ndarray) -> np.ndarray:
    """uint8 e4m3 codes -> float32: sign, 4 exponent bits (bias 7), 3 mantissa bits; exponent 0 is subnormal (m / 8 * 2^-6);
    0x7F / 0xFF are NaN (the format has no infinities)."""
    c = np.asarray(code).astype(np.int32)
    e, m = (c >> 3) & 15, c & 7
    mag = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1.0 + m / 8.0) * np.exp2(e - 7.0))
    mag = np.where((e == 15) & (m == 7), np.nan, mag)
    return np.where(c & 128, -mag, mag).astype(F32)


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """float values with |x| <= 448 -> uint8 e4m3 codes, round to nearest, ties to even (on the 3-bit mantissa, or on the
    subnormal grid of 2^-9 below 2^-6)."""
    x = np.asarray(x, dtype=np.float64)
    if x.size and np.abs(x).max() > E4M3_MAX:
        raise ValueError("clamp to +-448 first")
    a = np.abs(x)
    _, ex = np.frexp(np.where(a > 0, a, 1.0))                  # a = f * 2^ex, 0.5 <= f < 1  ->  floor(log2 a) = ex - 1
    e = np.maximum(ex - 1, -6)                                  # below 2^-6 the spacing stays that of the smallest normal binade
    q = np.rint(a / np.exp2(e - 3.0))                           # multiples of the spacing 2^(e-3); np.rint rounds ties to even
    carry = q >= 16                                             # rounded up into the next binade
    e = np.where(carry, e + 1, e)
    q = np.where(carry, 8, q).astype(np.int64)
    code = np.where(q < 8, q, ((e + 7) << 3) | (q - 8)).astype(np.int64)   # q < 8: subnormal (exponent field 0)
    return (code | np.where(np.signbit(x), 128, 0)).astype(np.uint8)


def quant_e4m3(t: np.ndarray):
    """Per-row fp8 quantisation in the dtype of ``t`` (fp16 on the path), the symmetric integer rule with 448 for the upper code:
    ``scale = max|row| / 448`` (zero rows: 1), ``codes = e4m3(clamp(row / scale, +-448))``.  Returns (codes uint8, scale [rows, 1])."""
    dt = t.dtype
    r = t.reshape(-1, t.shape[-1])
    scale = (np.abs(r).max(axis=-1, keepdims=True) / dt.type(E4M3_MAX)).astype(dt)
    scale = np.where(scale == 0, dt.type(1), scale).astype(dt)
    q = np.clip((r / scale).astype(dt), dt.type(-E4M3_MAX), dt.type(E4M3_MAX))
    return e4m3_encode(q.astype(np.float64)).reshape(t.shape), scale


def fp8_gemm(ca: np.ndarray, cb: np.ndarray) -> np.ndarray:
    """``acc[m, n] = sum_k value(ca[m, k]) * value(cb[n, k])`` for e4m3 codes, as float32.  Every product is exact in fp32; the
    matrix instruction adds the products of a step in an order and an alignment of its own (measured: about 2^-16 of the largest sum
    away from this float64 sum rounded once), so comparisons with it carry a tolerance."""
    return (e4m3_decode(ca).astype(np.float64) @ e4m3_decode(cb).astype(np.float64).T).astype(F32)


def linear_block_fp8(x: np.ndarray, w: np.ndarray, rotate: bool):
    """One w8a8 block in fp8: activations optionally rotated, per-token e4m3; weights per-channel e4m3; fp32 sums; the w-a epilogue.
    Returns (out fp16, out of the fake-quant path fp16: dequantised operands multiplied in float64)."""
    xr = online_hadamard(x) if rotate else x
    ca, sa = quant_e4m3(xr)
    cb, sb = quant_e4m3(w)
    acc = fp8_gemm(ca, cb)
    out = (acc * (sa.reshape(-1, 1).astype(F32) * sb.reshape(1, -1).astype(F32))).astype(F32).astype(F16)
    xq = (e4m3_decode(ca).astype(F16) * sa.astype(F16)).astype(F16)
    wq = (e4m3_decode(cb).astype(F16) * sb.astype(F16)).astype(F16)
    return out, gemm_fakequant(xq, wq)


# --------------------------------------------------------------------------------------------
# Tile scheduler  (mxmoe/kernels/src/include/tile_scheduler.cuh:5-50, kernel_sketch.py:87-101)
# --------------------------------------------------------------------------------------------
def tile_prefix(problem_mn, tile_mn):
    """Inclusive prefix sum of ``ceil(M/BM) * ceil(N/BN)`` per problem (kernel_sketch.py:89-101)."""
    tot, out = 0, []
    for (m, n), (bm, bn) in zip(problem_mn, tile_mn):
        tot += -(-m // bm) * -(-n // bn)
        out.append(tot)
    return out


def tile_to_problem(tile_idx: int, prefix, problem_mn, tile_mn):
    """tile_scheduler.cuh:25-49: first problem with ``prefix[i] > tile_idx``; local index -> (idx // grid_n, idx % grid_n).

    Returns ``(-1, 0, 0)`` past the end, else ``(problem, tile_m, tile_n)`` (x = row tile, y = column tile).
    """
    if not prefix or tile_idx >= prefix[-1]:
        return -1, 0, 0
    p = next(i for i, s in enumerate(prefix) if tile_idx < s)
    local = tile_idx - (prefix[p - 1] if p else 0)
    grid_n = -(-problem_mn[p][1] // tile_mn[p][1])
    return p, local // grid_n, local % grid_n


# --------------------------------------------------------------------------------------------
# Whole-layer fake-quant path (what the CPU baseline times) and the integer path next to it
# --------------------------------------------------------------------------------------------
def quant_weight(w: np.ndarray, w_bits: int, gsize: int, sym: bool):
    """RTN weight quantisation = ``quant_minmax`` on the ``[N, K]`` weight rows (quant.py:913 / quantize.cuh:218-279)."""
    return quant_minmax(w, w_bits, gsize, sym)


def linear_block(x: np.ndarray, w: np.ndarray, qp, rotate: bool):
    """One linear block of one expert in one format ``qp = (a_bits, w_bits, gsize, sym)``.

    Returns ``(out_kernel fp16, out_fakequant fp16, acc int32 | None)``:
    * w-a formats (a_bits < 16): activations optionally rotated (``online_hadamard``), per-token sym
      quantised; weights per-channel sym RTN; ``acc = int_gemm``; ``out_kernel = epilogue_wxax``;
      ``out_fakequant = gemm_fakequant(dequant(xq), dequant(wq))`` (quant.py:126-130 path).
    * weight-only (a_bits == 16, w_bits < 16): ``out = x @ fake_quant(w).T``; fp16: plain GEMM.
    """
    a_bits, w_bits, g, sym = qp
    if a_bits < 16 and g > 0:
        # group-quantised on both sides (w4a4_g128_sym): acc is the [G, M, N] stack of per-group accumulators
        xr = online_hadamard(x) if rotate else x
        qa, sa, _ = quant_minmax(xr, a_bits, g, True)
        qb, sb, _ = quant_minmax(w, w_bits, g, True)
        acc = int_gemm_grouped(qa, qb, g)
        out_k, _ = epilogue_grouped(acc, sa.reshape(x.shape[0], -1), sb.reshape(w.shape[0], -1))
        out_f = gemm_fakequant(dequant(qa, sa, 0 * sa, g), dequant(qb, sb, 0 * sb, g))
        return out_k, out_f, acc
    if a_bits < 16:
        xr = online_hadamard(x) if rotate else x
        qa, sa, _ = quant_minmax(xr, a_bits, -1, True)
        qb, sb, _ = quant_minmax(w, w_bits, -1, True)
        acc = int_gemm(qa, qb)
        out_k = epilogue_wxax(acc, sa.reshape(-1), sb.reshape(-1))
        out_f = gemm_fakequant(dequant(qa, sa, 0 * sa, -1), dequant(qb, sb, 0 * sb, -1))
        return out_k, out_f, acc
    wq = fake_quant(w, w_bits, g, sym) if w_bits < 16 else w
    out = gemm_fakequant(x, wq)
    return out, out, None


def unpermute_combine(down_rows, src_slot, topk_weights, shared=None):
    """The step after the down projection: out[t] = sum_k w[t, k] * down(row of (t, k)) + shared[t].

    The reference only has an empty stub for it (`gg_unpermute_out`, mxmoe/kernels/src/ref_bind.cu:66); the arithmetic fixed here is
    fp32, slots in ascending k, every product and every sum rounded to fp32, one final rounding to fp16.  `src_slot[r]` is the
    flattened (token, slot) index of sorted row r (rows of dropped expert ids simply do not appear).
    Pinned by: one-hot weights return the routed row itself, a dense float64 evaluation to fp16 tolerance, invariance under the
    order of the sorted rows (tests/test_oracle_host.py)."""
    w = np.asarray(topk_weights, dtype=np.float32)
    t, k = w.shape
    rows = np.asarray(down_rows, dtype=np.float16)
    row_of = np.full(t * k, -1, dtype=np.int64)
    row_of[np.asarray(src_slot, dtype=np.int64)] = np.arange(len(src_slot))
    acc = np.zeros((t, rows.shape[1]), dtype=np.float32)
    for j in range(k):
        r = row_of.reshape(t, k)[:, j]
        ok = r >= 0
        prod = (w[ok, j][:, None] * rows[r[ok]].astype(np.float32)).astype(np.float32)
        acc[ok] = (acc[ok] + prod).astype(np.float32)
    if shared is not None:
        acc = (acc + np.asarray(shared, dtype=np.float16).astype(np.float32)).astype(np.float32)
    return acc.astype(np.float16)

