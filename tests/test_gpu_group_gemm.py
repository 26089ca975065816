"""GPU parity of the fused GroupGEMM (through the C-ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
F16 = np.float16
DEV = "cuda"


def _rel(a, b):
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-6)


def _wxax_problem(rng, m, n, k, bits, rotate=False, bf6=False):
    """`bf6`: int4 operands as bf6 fragments, the layout of the kernels whose w4a4 tiles run on the 6-bit float matrix path."""
    from mxmoe_amd import pack

    x = rng.standard_normal((m, k)).astype(F16)
    w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
    qa, sa, _ = O.quant_minmax(x, bits, -1, True)
    qb, sb, _ = O.quant_minmax(w, bits, -1, True)
    ta, tb = torch.from_numpy(qa.astype(np.int8)), torch.from_numpy(qb.astype(np.int8))
    acc = O.int_gemm(qa, qb)
    if bits == 4 and bf6:
        ta, tb = pack.pack_bf6_fragments(ta), pack.pack_bf6_fragments(tb)
    else:
        if bits == 4:
            ta, tb = pack.pack_int4_k(ta), pack.pack_int4_k(tb)
        tb = pack.pack_wxax_fragments(tb)                  # weights travel in MFMA fragment order
    return dict(A=ta.to(DEV), B=tb.to(DEV), sa=torch.from_numpy(sa.reshape(-1)).to(DEV), sb=torch.from_numpy(sb.reshape(-1)).to(DEV),
                acc=acc, out=O.epilogue_wxax(acc, sa.reshape(-1), sb.reshape(-1)),
                fq=O.gemm_fakequant(O.dequant(qa, sa, 0 * sa, -1), O.dequant(qb, sb, 0 * sb, -1)),
                size=(m, n, k), q=(bits, bits, -1, True))


def _launch(probs, kernel_id=-1, dump=True):
    from mxmoe_amd.group_gemm import GroupGemmLaunch

    Cs = [torch.full((p["size"][0], p["size"][1]), float("nan"), dtype=torch.float16, device=DEV) for p in probs]
    accs = [torch.zeros((p["size"][0], p["size"][1]), dtype=torch.int32, device=DEV) for p in probs] if dump else None
    g = GroupGemmLaunch([p["A"] for p in probs], [p["B"] for p in probs], [p.get("sa") for p in probs], [p.get("sb") for p in probs],
                        Cs, [p["size"] for p in probs], [p["q"] for p in probs], kernel_id=kernel_id, acc=accs)
    g.run()
    torch.cuda.synchronize()
    return g, [c.cpu().numpy() for c in Cs], ([a.cpu().numpy() for a in accs] if dump else None)


def test_wxax_mixed_launch_bit_exact_accumulators():
    rng = np.random.default_rng(0)
    shapes = [(1, 256, 128, 4), (31, 512, 256, 8), (33, 384, 1408, 4), (130, 256, 256, 8), (300, 768, 384, 4),
              (64, 2816, 2048, 4), (129, 2048, 1408, 8), (17, 264, 128, 8)]
    probs = [_wxax_problem(rng, m, n, k, b) for (m, n, k, b) in shapes]
    g, outs, accs = _launch(probs)
    kid, branches, tiles = g.plan()
    print("kernel", kid, "branches", branches, "tiles", tiles)
    for p, out, acc in zip(probs, outs, accs):
        assert np.array_equal(acc, p["acc"]), f"int32 accumulators differ for {p['size']} {p['q']}"
        assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), f"fp16 epilogue differs for {p['size']}"
        assert _rel(out, p["fq"]) <= 1e-2                                  # tolerance of the fake-quant comparison


@pytest.mark.parametrize("kernel", ["groupgemm_hz_fused_wxax_b6", "groupgemm_hz_fused_all_b6"])
def test_w4a4_on_the_bf6_matrix_path_bit_exact(kernel):
    """The kernels whose w4a4 tiles run on v_mfma_scale_f32_32x32x64_f8f6f4 (int4 values as bf6 fragments on both sides), mixed
    with w8a8 in one launch: the accumulators are the integer products and the fp16 outputs the integer tiles' epilogue, bit for
    bit, for ragged row counts (every tile height, segments, rows past the last block), channel counts that are no multiple of a
    tile or of a fragment, and K from the shortest the tile takes to Qwen's and Mixtral's."""
    from mxmoe_amd import _lib

    kid = _lib.load().mxmoe_find_kernel(kernel.encode())
    assert kid >= 0
    rng = np.random.default_rng(21)
    shapes = [(1, 256, 256, 4), (31, 512, 256, 8), (33, 384, 1408, 4), (130, 256, 256, 8), (300, 768, 384, 4), (64, 2816, 2048, 4),
              (129, 2048, 1408, 8), (17, 264, 256, 4), (546, 520, 512, 4), (97, 1024, 4096, 4), (32, 256, 128 * 5, 4)]
    probs = [_wxax_problem(rng, m, n, k, b, bf6=True) for (m, n, k, b) in shapes]
    for rep in range(3):
        g, outs, accs = _launch(probs, kernel_id=kid)
        for p, out, acc in zip(probs, outs, accs):
            assert np.array_equal(acc, p["acc"]), f"launch {rep}: accumulators differ for {p['size']} {p['q']}"
            assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), f"launch {rep}: fp16 epilogue differs for {p['size']}"
            assert _rel(out, p["fq"]) <= 1e-2
    # extreme codes: every product at its largest magnitude, K = 14336 (sums of 64 * K stay far below 2^24)
    m, n, k = 40, 256, 14336
    qa = np.where(rng.random((m, k)) < 0.5, -7, 7).astype(np.int8)
    qb = np.where(rng.random((n, k)) < 0.5, -7, 7).astype(np.int8)
    qb[::2] = 7
    qa[1::2] = 7
    from mxmoe_amd import pack

    one = np.ones(max(m, n), F16)
    p = dict(A=pack.pack_bf6_fragments(torch.from_numpy(qa)).to(DEV), B=pack.pack_bf6_fragments(torch.from_numpy(qb)).to(DEV), sa=torch.from_numpy(one[:m].copy()).to(DEV),
             sb=torch.from_numpy(one[:n].copy()).to(DEV), size=(m, n, k), q=(4, 4, -1, True))
    _, _, accs = _launch([p], kernel_id=kid)
    assert np.array_equal(accs[0], O.int_gemm(qa, qb))
    # values the quantiser never emits but the format holds (-8, +8), and one-hot operands that pin which (row, k) a lane's bits stand for
    m, n, k = 96, 256, 512
    qa, qb = rng.integers(-8, 9, (m, k)).astype(np.int8), rng.integers(-8, 9, (n, k)).astype(np.int8)
    ha, hb = np.zeros((m, k), np.int8), rng.integers(-8, 9, (n, k)).astype(np.int8)
    for r in range(m):
        ha[r, (37 * r + 11) % k] = (r % 15) - 7
    for a_, b_ in ((qa, qb), (ha, hb)):
        p = dict(A=pack.pack_bf6_fragments(torch.from_numpy(a_)).to(DEV), B=pack.pack_bf6_fragments(torch.from_numpy(b_)).to(DEV), sa=torch.from_numpy(one[:m].copy()).to(DEV),
                 sb=torch.from_numpy(one[:n].copy()).to(DEV), size=(m, n, k), q=(4, 4, -1, True))
        _, _, accs = _launch([p], kernel_id=kid)
        assert np.array_equal(accs[0], O.int_gemm(a_, b_))
    # shapes the tile does not take are refused on the host
    bad = _wxax_problem(rng, 4, 256, 256, 4, bf6=True)
    bad["size"] = (4, 256, 128)
    with pytest.raises(RuntimeError, match="not supported by tile"):
        _launch([bad], kernel_id=kid)


def test_w8a8_in_fp8_e4m3_next_to_w4a4():
    """The kernel whose w8a8 tiles run the fp8 matrix instruction (the reference's w8a8_g-1_sym_E4M3, tile_config.py:45): e4m3
    codes on both sides, fp32 sums.  The instruction adds the products of a step in an order and an alignment of its own (sums
    come out about 2^-16 of the largest sum away from the float64 sum), so the fp32 sums are compared within 2e-4 of the largest,
    the fp16 outputs within 1e-3 of the oracle's and 1e-2 of the fake-quant path; the w4a4 problems of the same launch stay bit-exact."""
    from mxmoe_amd import _lib, pack

    lib = _lib.load()
    kid = lib.mxmoe_find_kernel(b"groupgemm_hz_fused_wxax_e4m3")
    assert kid >= 0 and "w8a8_g-1_sym_E4M3" in lib.mxmoe_kernel_name(kid).decode()
    rng = np.random.default_rng(41)
    probs = []
    for (m, n, k) in [(1, 256, 64), (31, 512, 256), (129, 2048, 1408), (300, 264, 384), (64, 2816, 2048)]:
        x = rng.standard_normal((m, k)).astype(F16)
        w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
        ca, sa = O.quant_e4m3(x)
        cb, sb = O.quant_e4m3(w)
        acc = O.fp8_gemm(ca, cb)
        out, fq = O.linear_block_fp8(x, w, False)
        probs.append(dict(A=torch.from_numpy(ca).to(DEV), B=pack.pack_wxax_fragments(torch.from_numpy(cb)).to(DEV), sa=torch.from_numpy(sa.reshape(-1)).to(DEV),
                          sb=torch.from_numpy(sb.reshape(-1)).to(DEV), acc32=acc, out=out, fq=fq, size=(m, n, k), q=(8, 8, -1, True)))
    probs.insert(2, _wxax_problem(rng, 70, 512, 256, 4))
    _, outs, accs = _launch(probs, kernel_id=kid)
    for p, out, acc in zip(probs, outs, accs):
        if "acc32" in p:
            got = acc.view(np.float32)
            assert np.abs(got - p["acc32"]).max() <= 2e-4 * np.abs(p["acc32"]).max() + 1e-6, p["size"]
            assert np.isfinite(out).all() and _rel(out, p["out"]) <= 1e-3 and _rel(out, p["fq"]) <= 1e-2, (p["size"], _rel(out, p["out"]))
        else:
            assert np.array_equal(acc, p["acc"]) and np.array_equal(out.view(np.uint16), p["out"].view(np.uint16))


def test_wxax_empty_and_single_row_problems():
    rng = np.random.default_rng(1)
    probs = [_wxax_problem(rng, m, 256, 128, b) for (m, b) in [(5, 8), (1, 4)]]
    empty = dict(probs[0])
    empty.update(A=torch.zeros((0, 128), dtype=torch.int8, device=DEV), sa=torch.zeros(0, dtype=torch.float16, device=DEV), size=(0, 256, 128))
    g, outs, accs = _launch([probs[0], empty, probs[1]])
    assert np.array_equal(accs[0], probs[0]["acc"]) and np.array_equal(accs[2], probs[1]["acc"])
    assert outs[1].shape == (0, 256)


def test_wxax_few_row_problems_every_wave_every_launch():
    """Problems of at most 32 rows (the 32-row tile, whose K slices are the shortest in time) with many column tiles, launched
    repeatedly: the accumulators of all four waves' columns must be exact on every launch.  A fragment register that the compiler
    copied before its hand-tracked load had landed showed up exactly here, as occasional stale weights in some waves' columns."""
    rng = np.random.default_rng(11)
    shapes = [(13, 3584, 512, 4), (7, 2048, 256, 8), (32, 1024, 128, 4), (1, 512, 1024, 8), (29, 2816, 2048, 4), (3, 2048, 1408, 8)]
    probs = [_wxax_problem(rng, m, n, k, b) for (m, n, k, b) in shapes]
    for kid in (-1, None):
        if kid is None:
            from mxmoe_amd import _lib

            kid = _lib.load().mxmoe_find_kernel(b"groupgemm_hz_fused_all")
            assert kid >= 0
        for rep in range(6):
            _, outs, accs = _launch(probs, kernel_id=kid)
            for p, out, acc in zip(probs, outs, accs):
                assert np.array_equal(acc, p["acc"]), f"launch {rep}, kernel {kid}: int32 accumulators differ for {p['size']} {p['q']}"
                assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16))


def test_more_problems_than_one_launch_holds():
    """A problem list longer than one launch's table (120 problems) runs as several launches; empty problems in between are skipped."""
    rng = np.random.default_rng(12)
    probs = []
    for i in range(150):
        m = [0, 1, 5, 33, 64][i % 5]
        b = 4 if i % 2 else 8
        p = _wxax_problem(rng, max(m, 1), 256, 128, b)
        if m == 0:
            p.update(A=torch.zeros((0, 128 if b == 8 else 64), dtype=torch.int8, device=DEV), sa=torch.zeros(0, dtype=torch.float16, device=DEV),
                     size=(0, 256, 128), acc=p["acc"][:0], out=p["out"][:0])
        probs.append(p)
    _, outs, accs = _launch(probs)
    for i, (p, out, acc) in enumerate(zip(probs, outs, accs)):
        assert np.array_equal(acc, p["acc"]), f"problem {i} {p['size']}"
        assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), f"problem {i} {p['size']}"


def _grouped_problem(rng, m, n, k):
    """w4a4_g128_sym: codes and group scales from the oracle quantiser, expected fp32 sums and fp16 outputs from its epilogue."""
    from mxmoe_amd import pack

    x = rng.standard_normal((m, k)).astype(F16)
    w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
    qa, sa, _ = O.quant_minmax(x, 4, 128, True)
    qb, sb, _ = O.quant_minmax(w, 4, 128, True)
    sa, sb = sa.reshape(m, k // 128), sb.reshape(n, k // 128)
    out, f32 = O.epilogue_grouped(O.int_gemm_grouped(qa, qb, 128), sa, sb)
    ta, tb = pack.pack_int4_k(torch.from_numpy(qa.astype(np.int8))), pack.pack_wxax_fragments(pack.pack_int4_k(torch.from_numpy(qb.astype(np.int8))))
    return dict(A=ta.to(DEV), B=tb.to(DEV), sa=torch.from_numpy(sa.copy()).to(DEV), sb=torch.from_numpy(np.ascontiguousarray(sb.T)).to(DEV),
                acc=f32.view(np.int32), out=out, fq=O.gemm_fakequant(O.dequant(qa, sa.reshape(-1, 1), 0 * sa.reshape(-1, 1), 128), O.dequant(qb, sb.reshape(-1, 1), 0 * sb.reshape(-1, 1), 128)),
                size=(m, n, k), q=(4, 4, 128, True))


def test_group_quantised_w4a4_bit_exact():
    """w4a4_g128_sym: the fp32 sums over the groups (dumped as bit patterns) and the fp16 outputs equal the oracle's bit for bit, alone
    and mixed with the per-channel formats in one launch."""
    rng = np.random.default_rng(13)
    shapes = [(1, 256, 128), (33, 384, 1408), (64, 2816, 2048), (130, 256, 256), (17, 264, 128), (300, 768, 384), (5, 2048, 1408)]
    probs = [_grouped_problem(rng, m, n, k) for (m, n, k) in shapes]
    _, outs, accs = _launch(probs)
    for p, out, acc in zip(probs, outs, accs):
        assert np.array_equal(acc, p["acc"]), f"fp32 group sums differ for {p['size']}"
        assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), f"fp16 outputs differ for {p['size']}"
        assert _rel(out, p["fq"]) <= 1e-2
    mixed = [probs[1], _wxax_problem(rng, 40, 512, 256, 4), probs[3], _wxax_problem(rng, 70, 256, 128, 8)]
    g, outs, accs = _launch(mixed)
    from mxmoe_amd import _lib

    assert b"fused_all" in _lib.load().mxmoe_kernel_name(g.plan()[0])
    for p, out, acc in zip(mixed, outs, accs):
        assert np.array_equal(acc, p["acc"]) and np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), p["size"]


def test_fp16_group_gemm():
    rng = np.random.default_rng(2)
    probs = []
    for (m, n, k) in [(34, 2816, 2048), (7, 512, 64), (200, 256, 1408), (128, 264, 32)]:
        x = rng.standard_normal((m, k)).astype(F16)
        w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
        probs.append(dict(A=torch.from_numpy(x).to(DEV), B=torch.from_numpy(w).to(DEV), ref=O.gemm_fp16(x, w), size=(m, n, k), q=(16, 16, -1, True)))
    _, outs, _ = _launch(probs, dump=False)
    for p, out in zip(probs, outs):
        assert _rel(out, p["ref"]) <= 1e-2, p["size"]
        assert _rel(out, p["ref"]) <= 2e-3                                 # fp32 accumulation: far inside the tolerance


def test_bf16_group_gemm():
    """The reference's `bf16` format (tile_config.py:42): bfloat16 operands and outputs on v_mfma_f32_32x32x16_bf16, kernel
    groupgemm_hz_fused_bf16 (chosen by name: its problems carry the QParams of fp16 ones).  Ragged problems within 1e-2 of the oracle,
    and small-integer operands, whose sums are exact whatever the order, bit for bit, ties of the output rounding included."""
    from mxmoe_amd import _lib, ops
    from mxmoe_amd.group_gemm import GroupGemmLaunch

    lib = _lib.load()
    kid = ops.select_kernel([(16, 16, -1, True)], bf16=True)
    assert lib.mxmoe_kernel_name(kid).decode().endswith("groupgemm_hz_fused_bf16") and ops.kernel_variants(lib, kid) == {0: 3}
    rng = np.random.default_rng(21)
    sizes = [(200, 264, 96), (1, 8, 32), (0, 64, 64), (33, 512, 1408), (129, 40, 2048)]
    As, Bs, Cs, refs = [], [], [], []
    for (m, n, k) in sizes:
        a = O.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
        b = O.bf16_round((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
        As.append(torch.from_numpy(O.bf16_bits(a).view(np.int16)).view(torch.float16).to(DEV))
        Bs.append(torch.from_numpy(O.bf16_bits(b).view(np.int16)).view(torch.float16).to(DEV))
        Cs.append(torch.full((m, n), float("nan"), dtype=torch.float16, device=DEV))
        refs.append(O.gemm_bf16(a, b))
    # exact case: integers up to 16 against 0 / 1 weights, and rows whose sums are the ties 257 -> 256 and 259 -> 260
    m, n, k = 64, 32, 64
    a = rng.integers(-16, 17, (m, k)).astype(np.float32)
    b = rng.integers(0, 2, (n, k)).astype(np.float32)
    a[0, :] = 0; a[0, 0], a[0, 1] = 256, 1
    a[1, :] = 0; a[1, 0], a[1, 1] = 258, 1
    b[:, 0] = b[:, 1] = 1
    As.append(torch.from_numpy(O.bf16_bits(a).view(np.int16)).view(torch.float16).to(DEV))
    Bs.append(torch.from_numpy(O.bf16_bits(b).view(np.int16)).view(torch.float16).to(DEV))
    Cs.append(torch.zeros((m, n), dtype=torch.float16, device=DEV))
    sizes.append((m, n, k))
    exact = O.bf16_round((a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    assert exact[0, 0] == 256.0 and exact[1, 0] == 260.0
    g = GroupGemmLaunch(As, Bs, None, None, Cs, sizes, [(16, 16, -1, True)] * len(sizes), kernel_id=kid, lib=lib)
    g.run()
    torch.cuda.synchronize()
    for c, ref, sz in zip(Cs[:-1], refs, sizes):
        if sz[0] == 0:
            continue
        got = c.view(torch.bfloat16).float().cpu().numpy()
        assert np.isfinite(got).all() and _rel(got, ref) <= 1e-2, sz
    got = O.bf16_from_bits(Cs[-1].cpu().numpy().view(np.uint16))
    assert np.array_equal(got.view(np.uint32), exact.view(np.uint32))


def test_weight_only_skinny():
    from mxmoe_amd.weights import quantize_and_pack

    rng = np.random.default_rng(3)
    probs = []
    for (m, n, k, bits, sym) in [(3, 2816, 2048, 4, False), (1, 256, 128, 3, False), (16, 128, 1408, 3, False), (32, 5632, 2048, 4, False),
                                 (5, 2048, 1408, 4, True), (19, 144, 256, 3, True), (4, 2816, 2048, 2, False), (16, 160, 384, 2, True)]:
        x = rng.standard_normal((m, k)).astype(F16)
        w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
        pw = quantize_and_pack(torch.from_numpy(w), (16, bits, 128, sym), keep_codes=True)
        q, s, z = O.quant_minmax(w, bits, 128, sym)
        codes = q.reshape(n, k) + ((1 << (bits - 1)) if sym else 0)
        assert np.array_equal(pw.q.numpy(), codes.astype(np.uint8))        # torch quantiser == oracle quantiser
        ref = O.gemm_fakequant(x, O.dequant(q, s, z, 128))
        probs.append(dict(A=torch.from_numpy(x).to(DEV), B=pw.data.to(DEV), sb=pw.scale.to(DEV), ref=ref, size=(m, n, k), q=(16, bits, 128, sym)))
    _, outs, _ = _launch(probs, dump=False)
    for p, out in zip(probs, outs):
        assert _rel(out, p["ref"]) <= 1e-2, (p["size"], p["q"], _rel(out, p["ref"]))


def test_weight_only_tiles_of_32_tokens():
    """Experts with 17 .. 32 tokens run the few-token tile with two blocks of 16 tokens per unpacked weight (from 33 tokens on the
    planner weighs two such tiles against the 128-token tile).  Its sums are formed in the same order as the 16-token tile's, so the outputs equal those of the kernel made
    of 16-token tiles bit for bit, besides staying within 1e-2 of the fake-quant path; ragged channel counts, K = 1408 (waves with 3, 3,
    3 and 2 k blocks), every bit width, per-channel scales."""
    import ctypes as C

    from mxmoe_amd import _lib
    from mxmoe_amd.weights import quantize_and_pack

    lib = _lib.load()
    rng = np.random.default_rng(17)
    cases = {"groupgemm_hz_fused_wo": [(17, 2816, 2048, 4, 128, False), (32, 144, 256, 3, 128, True), (31, 2048, 1408, 4, -1, False), (24, 160, 384, 2, 128, True),
                                        (32, 5632, 2048, 4, 128, False), (47, 256, 1408, 3, 128, False), (20, 128, 128, 2, -1, False), (3, 256, 256, 4, 128, False),
                                        (20, 256, 14336, 4, 128, False)],   # (the last: 14 passes per wave)
             "groupgemm_hz_fused_wo8": [(17, 256, 2048, 8, 128, False), (32, 2816, 1408, 8, -1, True), (25, 144, 256, 8, 128, True), (9, 128, 128, 8, 128, False)]}
    for kernel, shapes in cases.items():
        probs = []
        for (m, n, k, bits, gs, sym) in shapes:
            x = rng.standard_normal((m, k)).astype(F16)
            w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
            pw = quantize_and_pack(torch.from_numpy(w), (16, bits, gs, sym))
            q, s_, z = O.quant_minmax(w, bits, gs, sym)
            ref = O.gemm_fakequant(x, O.dequant(q, s_, z, gs))
            probs.append(dict(A=torch.from_numpy(x).to(DEV), B=pw.data.to(DEV), sb=pw.scale.to(DEV), ref=ref, size=(m, n, k), q=(16, bits, gs, sym)))
        kid = lib.mxmoe_find_kernel(kernel.encode())
        assert kid >= 0
        g, outs, _ = _launch(probs, kernel_id=kid, dump=False)
        _, branches, _ = g.plan()
        info = (C.c_int32 * 8)()
        bms = []
        for b in branches:
            assert lib.mxmoe_kernel_branch(kid, b, info) == 0
            bms.append(info[1])
        assert 32 in bms and 16 in bms, bms                                # the new tile is in use, next to the 16-token one
        for p, out in zip(probs, outs):
            assert np.isfinite(out).all() and _rel(out, p["ref"]) <= 1e-2, (p["size"], p["q"], _rel(out, p["ref"]))
        if kernel.endswith("_wo"):                                         # the same problems through 16-token tiles only
            few = lib.mxmoe_find_kernel(b"groupgemm_hz_fused_wo_skinny")
            _, outs16, _ = _launch(probs, kernel_id=few, dump=False)
            for p, a, b in zip(probs, outs, outs16):
                if p["size"][0] <= 32:    # (more rows go to the 128-token tile, which rounds every dequantised weight to fp16: other last bits)
                    assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), p["size"]


def test_weight_only_many_tokens():
    """Experts with many tokens run the 128 x 256 dequantise-to-fp16 MFMA tile (and the remainder rows the skinny one); channel
    counts that leave one or two of its four waves without channels are among the cases."""
    import ctypes as C

    from mxmoe_amd import _lib
    from mxmoe_amd.weights import quantize_and_pack

    rng = np.random.default_rng(5)
    probs = []
    for (m, n, k, bits, sym) in [(200, 256, 512, 4, False), (129, 384, 1408, 3, False), (64, 256, 128, 4, True), (300, 2816, 256, 3, True),
                                 (128, 192, 256, 4, False), (7, 256, 256, 4, False), (150, 256, 1408, 2, False), (200, 128, 256, 4, False)]:
        x = rng.standard_normal((m, k)).astype(F16)
        w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
        pw = quantize_and_pack(torch.from_numpy(w), (16, bits, 128, sym))
        q, s, z = O.quant_minmax(w, bits, 128, sym)
        ref = O.gemm_fakequant(x, O.dequant(q, s, z, 128))
        probs.append(dict(A=torch.from_numpy(x).to(DEV), B=pw.data.to(DEV), sb=pw.scale.to(DEV), ref=ref, size=(m, n, k), q=(16, bits, 128, sym)))
    g, outs, _ = _launch(probs, dump=False)
    kid, branches, _ = g.plan()
    lib = _lib.load()
    info = (C.c_int32 * 8)()
    bms = []
    for b in branches:
        assert lib.mxmoe_kernel_branch(kid, b, info) == 0
        bms.append(info[1])
    assert bms[:5] == [128] * 5 and bms[5] == 16 and bms[6:] == [128, 128], bms
    for p, out in zip(probs, outs):
        assert np.isfinite(out).all()
        assert _rel(out, p["ref"]) <= 1e-2, (p["size"], p["q"], _rel(out, p["ref"]))


def test_per_channel_and_eight_bit_weight_only_formats():
    """The weight-only formats of the reference's generator beyond group 128 (mxmoe/kernels/tile_config.py:40-59; the kernel its
    operator wires in is w4a16 per channel, asymmetric: mxmoe/kernels/src/ref_bind.cu:412-424, hz_fused.cuh:428-434): one scale per
    channel (group size -1) for 4 / 3 / 2 bits, and 8-bit weights with either group size; few-token and many-token tiles, symmetric
    and asymmetric, mixed in one launch per kernel.  Outputs within 1e-2 of the fake-quant path."""
    from mxmoe_amd.weights import quantize_and_pack

    rng = np.random.default_rng(31)
    cases = [(3, 2816, 2048, 4, -1, False), (200, 256, 512, 4, -1, False), (16, 128, 1408, 3, -1, False), (150, 384, 1408, 2, -1, True), (5, 2048, 1408, 4, -1, True),
             (3, 2816, 2048, 8, 128, False), (1, 256, 128, 8, -1, False), (200, 256, 512, 8, 128, True), (129, 384, 1408, 8, -1, True), (16, 160, 384, 8, 128, False),
             (300, 2048, 1408, 8, -1, False)]
    probs = []
    for (m, n, k, bits, g, sym) in cases:
        x = rng.standard_normal((m, k)).astype(F16)
        w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
        pw = quantize_and_pack(torch.from_numpy(w), (16, bits, g, sym), keep_codes=True)
        q, s, z = O.quant_minmax(w, bits, g, sym)
        codes = q.reshape(n, k) + ((1 << (bits - 1)) if sym else 0)
        assert np.array_equal(pw.q.numpy(), codes.astype(np.uint8))        # torch quantiser == oracle quantiser
        probs.append(dict(A=torch.from_numpy(x).to(DEV), B=pw.data.to(DEV), sb=pw.scale.to(DEV), ref=O.gemm_fakequant(x, O.dequant(q, s, z, g)),
                          size=(m, n, k), q=(16, bits, g, sym)))
    for group in ([p for p in probs if p["q"][1] != 8], [p for p in probs if p["q"][1] == 8]):
        g_, outs, _ = _launch(group, dump=False)
        for p, out in zip(group, outs):
            assert np.isfinite(out).all() and _rel(out, p["ref"]) <= 1e-2, (p["size"], p["q"], _rel(out, p["ref"]))


def _any_problem(rng, fmt, m, n, k):
    from mxmoe_amd.weights import quantize_and_pack

    if fmt in ("w4a4", "w8a8"):
        return _wxax_problem(rng, m, n, k, 4 if fmt == "w4a4" else 8)
    if fmt == "w4a4g":
        return _grouped_problem(rng, m, n, k)
    x = rng.standard_normal((m, k)).astype(F16)
    w = (rng.standard_normal((n, k)) * 0.02).astype(F16)
    if fmt == "fp16":
        return dict(A=torch.from_numpy(x).to(DEV), B=torch.from_numpy(w).to(DEV), ref=O.gemm_fp16(x, w), size=(m, n, k), q=(16, 16, -1, True))
    bits, sym = int(fmt[1]), fmt.endswith("s")
    pw = quantize_and_pack(torch.from_numpy(w), (16, bits, 128, sym))
    q, sc, z = O.quant_minmax(w, bits, 128, sym)
    return dict(A=torch.from_numpy(x).to(DEV), B=pw.data.to(DEV), sb=pw.scale.to(DEV), ref=O.gemm_fakequant(x, O.dequant(q, sc, z, 128)),
                size=(m, n, k), q=(16, bits, 128, sym))


@pytest.mark.parametrize("seed", [101, 102, 103])
def test_random_shapes_every_format_in_mixed_launches(seed):
    """Seeded sweep over ragged shapes: any M (empty problems, one row, tile sizes +- 1), N any multiple of the format's step (not of a
    tile), K any multiple of the format's slice, formats mixed in one launch.  Integer formats bit-exact, the others within 1e-2."""
    rng = np.random.default_rng(seed)
    k_step = {"w4a4": 128, "w8a8": 64, "w4a4g": 128, "fp16": 32, "w4a": 128, "w3a": 128, "w2s": 128, "w4s": 128}
    n_step = {"w4a4": 8, "w8a8": 8, "w4a4g": 8, "fp16": 8}
    fmts = list(k_step)
    probs = []
    for _ in range(14):
        fmt = fmts[int(rng.integers(len(fmts)))]
        m = int(rng.choice([1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 257]))
        n = n_step.get(fmt, 16) * int(rng.integers(1, 60))
        k = k_step[fmt] * int(rng.integers(1, 1 + 1536 // k_step[fmt]))
        probs.append(_any_problem(rng, fmt, m, n, k))
    empty = dict(probs[0])
    empty.update(A=torch.zeros((0, 8), dtype=torch.int8, device=DEV), sa=torch.zeros(0, dtype=torch.float16, device=DEV), size=(0,) + probs[0]["size"][1:])
    probs.insert(3, empty)
    g, outs, accs = _launch(probs)
    print("seed", seed, "kernel", g.plan()[0], [(p["q"], p["size"]) for p in probs])
    for i, (p, out, acc) in enumerate(zip(probs, outs, accs)):
        if p["size"][0] == 0:
            continue
        if "acc" in p:
            assert np.array_equal(acc, p["acc"]), (i, p["size"], p["q"])
            assert np.array_equal(out.view(np.uint16), p["out"].view(np.uint16)), (i, p["size"], p["q"])
        else:
            assert np.isfinite(out).all() and _rel(out, p["ref"]) <= 1e-2, (i, p["size"], p["q"], _rel(out, p["ref"]))


def test_unsupported_format_raises_reference_message():
    rng = np.random.default_rng(4)
    p = _wxax_problem(rng, 4, 256, 128, 8)
    p["q"] = (8, 4, -1, True)
    with pytest.raises(RuntimeError, match="quant type not supported"):
        _launch([p])
    p = _wxax_problem(rng, 4, 256, 128, 8)
    p["size"] = (4, 256, 100)
    with pytest.raises(RuntimeError, match="not supported by tile"):
        _launch([p])
