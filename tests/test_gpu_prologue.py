"""GPU parity of the prologue kernels (permutation, act-quant with Hadamard, SiLU*up-quant) and of the whole layer
chained through the `mxmoe_ops`-style operators, against the CPU oracle.  Integer codes and scales must be bit-exact."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
F16 = np.float16
DEV = "cuda"


def _ids(rng, t, e, k):
    return np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)


def test_permutation_matches_oracle_and_is_stable():
    from mxmoe_amd import ops

    rng = np.random.default_rng(0)
    for (t, e, k) in [(1, 4, 2), (37, 7, 3), (300, 60, 4), (2048, 64, 6), (513, 8, 2), (12000, 64, 6)]:   # (the last: beyond the scan-less path)
        ids = _ids(rng, t, e, k)
        if e > 5:
            ids[ids == 3] = 5 if k == 1 else ids[ids == 3]                  # keep ids valid
        dst, perm, slot, recv = ops.build_permutation(torch.from_numpy(ids).to(DEV), e)
        torch.cuda.synchronize()
        o_dst, o_perm, o_slot, o_recv = O.permute_by_expert(ids, e)
        assert np.array_equal(dst.cpu().numpy(), o_dst)
        assert np.array_equal(perm.cpu().numpy(), o_perm)
        assert np.array_equal(slot.cpu().numpy(), o_slot)
        assert np.array_equal(recv.cpu().numpy(), o_recv)


def test_permutation_with_inverse_map_small_and_large_and_dropped_ids():
    """mxmoe_build_permutation_inv: the reference's four outputs plus row_of_slot, the inverse map the combine reads; sizes on both
    sides of the single-launch path (at most 256 entries), ids out of range dropped (-1 in the inverse map)."""
    from mxmoe_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(3)
    stream = torch.cuda.current_stream().cuda_stream
    for (t, e, k) in [(1, 4, 2), (32, 64, 6), (42, 7, 6), (43, 7, 6), (64, 4, 4), (65, 4, 4), (700, 60, 4), (3000, 256, 8)]:   # (the last: with the scan kernel)
        ids = _ids(rng, t, e, k)
        ids[rng.random(ids.shape) < 0.15] = e + 2                            # dropped entries
        if t > 3:
            ids[1, 0] = -1
        total = t * k
        d_ids = torch.from_numpy(ids).to(DEV)
        dst = torch.full((total,), -7, dtype=torch.int32, device=DEV)
        perm = torch.full((total,), -7, dtype=torch.int64, device=DEV)
        slot = torch.full((total,), -7, dtype=torch.int64, device=DEV)
        recv = torch.empty(e, dtype=torch.int64, device=DEV)
        inv = torch.full((total,), -7, dtype=torch.int32, device=DEV)
        ws = torch.empty(max(lib.mxmoe_permute_workspace_bytes(total, e), 16), dtype=torch.uint8, device=DEV)
        for _ in range(2):                                                   # a second call over the same buffers gives the same result
            _lib.check(lib, lib.mxmoe_build_permutation_inv(d_ids.data_ptr(), t, k, e, dst.data_ptr(), perm.data_ptr(), slot.data_ptr(), recv.data_ptr(),
                                                            inv.data_ptr(), ws.data_ptr(), stream))
        torch.cuda.synchronize()
        flat = ids.reshape(-1).astype(np.int64)
        keep = np.nonzero((flat >= 0) & (flat < e))[0]                      # the oracle's stable sort, over the entries that are routed
        order = keep[np.argsort(flat[keep], kind="stable")]
        o_dst, o_perm, o_slot, o_recv = flat[order].astype(np.int32), order // k, order, np.bincount(flat[keep], minlength=e)
        if len(keep) == total:
            for a, b in zip((o_dst, o_perm, o_slot, o_recv), O.permute_by_expert(ids, e)):
                assert np.array_equal(a, b)
        r = len(o_dst)
        assert int(recv.sum()) == r
        assert np.array_equal(dst.cpu().numpy()[:r], o_dst) and np.array_equal(perm.cpu().numpy()[:r], o_perm)
        assert np.array_equal(slot.cpu().numpy()[:r], o_slot) and np.array_equal(recv.cpu().numpy(), o_recv)
        want = np.full(total, -1, np.int32)
        want[o_slot] = np.arange(r, dtype=np.int32)
        assert np.array_equal(inv.cpu().numpy(), want)


def _unpack(store_view, tag, n):
    raw = store_view.contiguous().view(torch.uint8).cpu().numpy().reshape(store_view.shape[0], -1)
    if tag == 1:
        return raw.view(np.int8)
    lo = (raw & 0xF).astype(np.int8)
    hi = (raw >> 4).astype(np.int8)
    q = np.stack([lo, hi], axis=-1).reshape(raw.shape[0], -1)
    return np.where(q >= 8, q - 16, q).astype(np.int8)


@pytest.mark.parametrize("k,rotate", [(2048, 1), (4096, 1), (256, 0), (2048, 2), (512, 1), (1024, 2), (2048, 0), (256, 1), (8192, 1), (2816, 2), (14336, 1),
                                      (1408, 1), (1408, 2), (224, 2), (96, 1)])
def test_quant_inp_act_bit_exact(k, rotate):
    from mxmoe_amd import ops

    rng = np.random.default_rng(k + rotate)
    t, e, topk, n_sh = 48, 6, 2, 1
    x = rng.standard_normal((t, k)).astype(F16)
    x[3] = 0                                                               # all-zero token: scale guard
    ids = _ids(rng, t, e, topk)
    ids[ids == 4] = 5 if False else ids[ids == 4]
    qp = [(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False), (4, 4, 128, True), (8, 8, -1, True), (16, 16, -1, True), (8, 8, -1, True)]
    if k % 128:                                                            # group-128 activations need rows that are multiples of 128
        qp[3] = (4, 4, -1, True)
    res = ops.quant_inp_act(torch.from_numpy(x).to(DEV), torch.from_numpy(ids).to(DEV), e, 1408, n_sh, qp, rotate=rotate)
    inp_list, scale_list, out_list, inp_store, scale_store, out_store, recv, perm, dst = res
    torch.cuda.synchronize()
    o_dst, o_perm, _, o_recv = O.permute_by_expert(ids, e)
    assert np.array_equal(recv.numpy(), o_recv)
    p = 0
    st = 0
    for ex in range(e + 1):
        m = t if ex == e else int(o_recv[ex])
        if m == 0:
            continue
        rows = x if ex == e else x[o_perm[st:st + m]]
        if ex < e:
            st += m
        a_bits = qp[ex][0]
        tag = O.act_tag(a_bits, qp[ex][2])
        rot = rotate == 2 or (rotate == 1 and tag != 0)
        xr = O.online_hadamard(rows) if rot else rows
        got = inp_list[p]
        assert out_list[p].shape == (m, 2 * 1408 * (n_sh if ex == e else 1))
        if tag == 0:
            assert np.array_equal(got.cpu().numpy().view(np.uint16), xr.view(np.uint16)), f"expert {ex} fp16 rows"
        else:
            q, s, _ = O.quant_minmax(xr, a_bits, 128 if tag == 3 else -1, True)   # tag 3: one scale per 128 values, [M, K / 128]
            assert np.array_equal(scale_list[p].cpu().numpy().view(np.uint16), s.reshape(-1).view(np.uint16)), f"expert {ex} scales"
            assert np.array_equal(_unpack(got, tag, k), q.astype(np.int8)), f"expert {ex} codes"
        p += 1
    assert p == len(inp_list)


@pytest.mark.parametrize("k,topk,rotate,n_sh", [(2048, 8, 1, 1), (512, 1, 2, 0), (4096, 3, 1, 0), (1024, 4, 0, 1), (2048, 4, 2, 1)])
def test_per_token_prologue_writes_the_same_bytes_as_the_per_row_one(k, topk, rotate, n_sh):
    """mxmoe_quant_act_tokens (a token quantised once per format among its destinations) against mxmoe_quant_act (once per
    destination row) over the same table: mixed formats (fp16 copies, int8, int4, int4 with group scales), expert ids out of range,
    an expert without rows, up to 8 slots per token.  The stores must match byte for byte."""
    from mxmoe_amd import _lib, ops

    lib = _lib.load()
    rng = np.random.default_rng(k + topk)
    t, e = 70, 10
    has_shared = n_sh > 0
    x = torch.from_numpy(rng.standard_normal((t, k)).astype(F16)).to(DEV)
    ids = _ids(rng, t, e, topk)
    ids[ids == 6] = 7 if topk == 1 else e + 3                              # expert 6 gets no rows; with top-k > 1 its slots are dropped
    ids[rng.random(ids.shape) < 0.1] = -1
    d_ids = torch.from_numpy(ids).to(DEV)
    fmts = [(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False), (4, 4, 128, True), (16, 16, -1, True)]
    qp = [fmts[i % len(fmts)] for i in range(e)] + [(8, 8, -1, True)]
    dst, perm, _slot, recv, inv = ops.build_permutation(d_ids, e, with_inverse=True)
    recv_cpu = recv.cpu()
    table, _rows, _isz, _ssz, _lds, io, so = ops._offsets(recv_cpu, t, e, has_shared, qp, k, k)
    d_table = table.to(DEV)
    routed = int(recv_cpu.sum())
    hk, hf, signs = ops.device_signs(k, DEV) if rotate else (1, 1, None)
    stream = torch.cuda.current_stream().cuda_stream
    stores = []
    for which in range(2):
        inp = torch.full((io,), 0x1234, dtype=torch.int16, device=DEV)
        sc = torch.full((max(so, 1),), 0x1234, dtype=torch.int16, device=DEV)
        if which == 0:
            _lib.check(lib, lib.mxmoe_quant_act(x.data_ptr(), inp.data_ptr(), sc.data_ptr(), dst.data_ptr(), perm.data_ptr(), d_table.data_ptr(), k, routed, t, e,
                                                int(has_shared), rotate, hk, hf, None if signs is None else signs.data_ptr(), stream))
        else:
            _lib.check(lib, lib.mxmoe_quant_act_tokens(x.data_ptr(), inp.data_ptr(), sc.data_ptr(), d_ids.data_ptr(), inv.data_ptr(), d_table.data_ptr(), k, t, topk, e,
                                                       int(has_shared), rotate, stream))
        torch.cuda.synchronize()
        stores.append((inp.cpu().numpy(), sc.cpu().numpy()))
    assert routed > 0 and (stores[0][0] != 0x1234).any()
    assert np.array_equal(stores[0][0], stores[1][0])
    assert np.array_equal(stores[0][1], stores[1][1])
    # shapes the per-token entry point refuses
    assert lib.mxmoe_quant_act_tokens(x.data_ptr(), inp.data_ptr(), sc.data_ptr(), d_ids.data_ptr(), inv.data_ptr(), d_table.data_ptr(), 1408, t, topk, e, 0, 1, stream) == 3
    assert lib.mxmoe_quant_act_tokens(x.data_ptr(), inp.data_ptr(), sc.data_ptr(), d_ids.data_ptr(), inv.data_ptr(), d_table.data_ptr(), k, t, 9, e, 0, 1, stream) == 3
    assert lib.mxmoe_quant_act_tokens(x.data_ptr(), inp.data_ptr(), sc.data_ptr(), d_ids.data_ptr(), inv.data_ptr(), d_table.data_ptr(), k, t, topk, e, 0, 5, stream) == 3


@pytest.mark.parametrize("n,n_sh,rotate", [(1408, 2, 2), (2048, 0, 1), (14336, 0, 1), (512, 1, 0), (1408, 0, 1), (1408, 1, 2), (224, 0, 2), (96, 1, 1)])
def test_silu_mul_then_quant_bit_exact(n, n_sh, rotate):
    from mxmoe_amd import ops

    rng = np.random.default_rng(n)
    t, e, topk = 12, 4, 2
    ids = _ids(rng, t, e, topk)
    o_dst, o_perm, _, o_recv = O.permute_by_expert(ids, e)
    r = t * topk
    gu = (rng.standard_normal((r, 2 * n)) * 2).astype(F16)
    gu_sh = (rng.standard_normal((t, 2 * n * max(n_sh, 1))) * 2).astype(F16)
    flat = np.concatenate([gu.reshape(-1), gu_sh.reshape(-1)]) if n_sh else gu.reshape(-1)
    qp = [(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False), (4, 4, 128, True), (8, 8, -1, True)]
    if n % 128:
        qp[3] = (8, 8, -1, True)
    res = ops.silu_mul_then_quant(torch.from_numpy(flat).to(DEV), int((o_recv != 0).sum()), e, 2048, n, n_sh, t, topk,
                                  torch.from_numpy(o_dst).to(DEV), torch.from_numpy(o_recv), qp, rotate=rotate)
    inp_list, scale_list, out_list = res[:3]
    torch.cuda.synchronize()
    p = st = 0
    for ex in range(e + (1 if n_sh else 0)):
        m = t if ex == e else int(o_recv[ex])
        if m == 0:
            continue
        src = gu_sh if ex == e else gu[st:st + m]
        if ex < e:
            st += m
        y = O.silu_mul(src)
        a_bits = qp[ex][0]
        tag = O.act_tag(a_bits, qp[ex][2])
        if rotate == 2 or (rotate == 1 and tag != 0):
            y = O.online_hadamard(y)
        got = inp_list[p]
        assert out_list[p].shape == (m, 2048)
        if tag == 0:
            assert np.array_equal(got.cpu().numpy().view(np.uint16), y.view(np.uint16)), f"expert {ex} fp16 rows"
        else:
            q, s, _ = O.quant_minmax(y, a_bits, 128 if tag == 3 else -1, True)
            assert np.array_equal(scale_list[p].cpu().numpy().view(np.uint16), s.reshape(-1).view(np.uint16)), f"expert {ex} scales"
            assert np.array_equal(_unpack(got, tag, y.shape[1]), q.astype(np.int8)), f"expert {ex} codes"
        p += 1


def _bf6_rows(view, m, k):
    """Codes of the m rows of an expert whose activations were written as bf6 fragments (tag 4)."""
    from mxmoe_amd import pack

    return pack.unpack_bf6_fragments(view.contiguous().view(torch.uint8).reshape(-1), m, k).cpu().numpy().astype(np.int8)


@pytest.mark.parametrize("k,rotate", [(2048, 1), (4096, 1), (256, 0), (1408, 1), (14336, 1), (2816, 2), (512, 2), (8192, 1)])
def test_quant_inp_act_writes_int4_codes_as_bf6_fragments(k, rotate):
    """With bf6=True the per-token int4 experts get their codes as bf6 fragments (the operand layout of the tiles on the 6-bit float
    matrix path): same scales and the same codes as the packed rows, value for value, in every row kernel (one row per wave with and
    without the dense stage, wide rows, the general kernel); rows per expert straddle the 32-row blocks; other formats are untouched."""
    from mxmoe_amd import ops

    rng = np.random.default_rng(k + rotate)
    t, e, topk, n_sh = 70, 5, 2, 1
    x = rng.standard_normal((t, k)).astype(F16)
    x[3] = 0
    ids = _ids(rng, t, e, topk)
    qp = [(4, 4, -1, True), (8, 8, -1, True), (4, 4, -1, True), (16, 16, -1, True), (4, 4, -1, True), (4, 4, -1, True)]
    res = ops.quant_inp_act(torch.from_numpy(x).to(DEV), torch.from_numpy(ids).to(DEV), e, 1408, n_sh, qp, rotate=rotate, bf6=True)
    inp_list, scale_list = res[:2]
    torch.cuda.synchronize()
    _, o_perm, _, o_recv = O.permute_by_expert(ids, e)
    p = st = 0
    for ex in range(e + 1):
        m = t if ex == e else int(o_recv[ex])
        if m == 0:
            continue
        rows = x if ex == e else x[o_perm[st:st + m]]
        if ex < e:
            st += m
        a_bits = qp[ex][0]
        tag = O.act_tag(a_bits, qp[ex][2])
        xr = O.online_hadamard(rows) if rotate == 2 or (rotate == 1 and tag != 0) else rows
        got = inp_list[p]
        if tag == 0:
            assert np.array_equal(got.cpu().numpy().view(np.uint16), xr.view(np.uint16))
        else:
            q, s, _ = O.quant_minmax(xr, a_bits, -1, True)
            assert np.array_equal(scale_list[p].cpu().numpy().view(np.uint16), s.reshape(-1).view(np.uint16)), f"expert {ex} scales"
            if a_bits == 4:
                assert got.shape == (-(-m // 32) * 32, k * 3 // 8)
                assert np.array_equal(_bf6_rows(got, m, k), q.astype(np.int8)), f"expert {ex} codes"
            else:
                assert np.array_equal(_unpack(got, tag, k), q.astype(np.int8)), f"expert {ex} codes"
        p += 1
    assert p == len(inp_list)


@pytest.mark.parametrize("n,n_sh,rotate", [(1408, 2, 1), (2048, 0, 1), (14336, 0, 1), (512, 1, 0)])
def test_silu_mul_then_quant_writes_bf6_fragments(n, n_sh, rotate):
    from mxmoe_amd import ops

    rng = np.random.default_rng(n + 7)
    t, e, topk = 40, 4, 2
    ids = _ids(rng, t, e, topk)
    o_dst, _, _, o_recv = O.permute_by_expert(ids, e)
    gu = (rng.standard_normal((t * topk, 2 * n)) * 2).astype(F16)
    gu_sh = (rng.standard_normal((t, 2 * n * max(n_sh, 1))) * 2).astype(F16)
    flat = np.concatenate([gu.reshape(-1), gu_sh.reshape(-1)]) if n_sh else gu.reshape(-1)
    qp = [(4, 4, -1, True), (8, 8, -1, True), (4, 4, -1, True), (4, 4, -1, True), (4, 4, -1, True)]
    res = ops.silu_mul_then_quant(torch.from_numpy(flat).to(DEV), int((o_recv != 0).sum()), e, 2048, n, n_sh, t, topk,
                                  torch.from_numpy(o_dst).to(DEV), torch.from_numpy(o_recv), qp, rotate=rotate, bf6=True)
    inp_list, scale_list = res[:2]
    torch.cuda.synchronize()
    p = st = 0
    for ex in range(e + (1 if n_sh else 0)):
        m = t if ex == e else int(o_recv[ex])
        if m == 0:
            continue
        src = gu_sh if ex == e else gu[st:st + m]
        if ex < e:
            st += m
        y = O.silu_mul(src)
        if rotate:
            y = O.online_hadamard(y)
        q, s, _ = O.quant_minmax(y, qp[ex][0], -1, True)
        assert np.array_equal(scale_list[p].cpu().numpy().view(np.uint16), s.reshape(-1).view(np.uint16)), f"expert {ex} scales"
        got = inp_list[p]
        codes = _bf6_rows(got, m, y.shape[1]) if qp[ex][0] == 4 else _unpack(got, 1, y.shape[1])
        assert np.array_equal(codes, q.astype(np.int8)), f"expert {ex} codes"
        p += 1


@pytest.mark.parametrize("k,rotate", [(2048, 1), (1408, 1), (14336, 1), (2816, 0)])
def test_quant_inp_act_writes_fp8_codes(k, rotate):
    """With fp8=True the per-token 8-bit experts get e4m3 codes and scales max / 448, bit for bit the oracle's, in every row kernel;
    the other formats are untouched."""
    from mxmoe_amd import ops

    rng = np.random.default_rng(k + 11)
    t, e, topk = 40, 4, 2
    x = (rng.standard_normal((t, k)) * rng.uniform(0.01, 20, (t, 1))).astype(F16)
    x[3] = 0
    ids = _ids(rng, t, e, topk)
    qp = [(8, 8, -1, True), (4, 4, -1, True), (8, 8, -1, True), (16, 16, -1, True), (8, 8, -1, True)]
    res = ops.quant_inp_act(torch.from_numpy(x).to(DEV), torch.from_numpy(ids).to(DEV), e, 1408, 1, qp, rotate=rotate, fp8=True)
    inp_list, scale_list = res[:2]
    torch.cuda.synchronize()
    _, o_perm, _, o_recv = O.permute_by_expert(ids, e)
    p = st = 0
    for ex in range(e + 1):
        m = t if ex == e else int(o_recv[ex])
        if m == 0:
            continue
        rows = x if ex == e else x[o_perm[st:st + m]]
        if ex < e:
            st += m
        tag = O.act_tag(qp[ex][0], qp[ex][2])
        xr = O.online_hadamard(rows) if rotate and tag != 0 else rows
        got = inp_list[p]
        if tag == 1:
            c, s_ = O.quant_e4m3(xr)
            assert np.array_equal(scale_list[p].cpu().numpy().view(np.uint16), s_.reshape(-1).view(np.uint16)), f"expert {ex} scales"
            assert np.array_equal(got.contiguous().view(torch.uint8).cpu().numpy().reshape(m, -1), c), f"expert {ex} codes"
        elif tag == 2:
            q, s_, _ = O.quant_minmax(xr, 4, -1, True)
            assert np.array_equal(_unpack(got, 2, k), q.astype(np.int8))
        p += 1


def test_unsupported_activation_format():
    from mxmoe_amd import ops

    x = torch.zeros((4, 256), dtype=torch.float16, device=DEV)
    ids = torch.zeros((4, 1), dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="quant type not supported"):
        ops.quant_inp_act(x, ids, 2, 128, 0, [(2, 2, -1, True), (8, 8, -1, True)])
