"""The one-pass host tables of a layer forward agree with the operator-by-operator builders of `ops.py` (which follow
mxmoe/kernels/src/ref_bind.cu:475-505 and 362-404) on random tokens-per-expert counts, empty experts and a shared expert included."""
import numpy as np
import pytest
import torch

from mxmoe_amd import layer_tables as LT
from mxmoe_amd import ops

FORMATS = [(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False), (16, 16, -1, True), (4, 4, 128, True), (16, 3, 128, False)]


@pytest.mark.parametrize("seed,has_shared", [(0, False), (1, True), (2, True), (3, False)])
def test_tables_match_the_operator_builders(seed, has_shared):
    rng = np.random.default_rng(seed)
    e, t, width, width_sh, n, n_sh = 9, 37, 256, 512, 384, 768
    et = e + (1 if has_shared else 0)
    qp = [FORMATS[i] for i in rng.integers(0, len(FORMATS), et)]
    recv = rng.integers(0, 40, e)
    recv[rng.integers(0, e, 3)] = 0                                   # empty experts
    rows = np.concatenate([recv, [t]]).astype(np.int64) if has_shared else recv.astype(np.int64)
    widths = [width] * e + ([width_sh] if has_shared else [])
    ns = [n] * e + ([n_sh] if has_shared else [])
    b_ptrs = [1000 * (i + 1) for i in range(et)]
    sb_ptrs = [0 if q[1] >= 16 else 77 * (i + 1) for i, q in enumerate(qp)]
    st = LT.static_block(qp, widths, ns, b_ptrs, sb_ptrs)
    bt = LT.block_tables(st, rows)

    table, rws, inp_sizes, scale_sizes, lds, io, so = ops._offsets(torch.from_numpy(recv), t, e, has_shared, qp, width, width_sh)
    assert np.array_equal(bt.table, table.numpy())
    assert (bt.inp_total, bt.scale_total) == (io, so)
    assert list(rows) == rws

    inp_store = torch.zeros(max(io, 1), dtype=torch.float16)
    scale_store = torch.zeros(max(so, 1), dtype=torch.float16)
    out_store = torch.zeros(max(bt.out_total, 1), dtype=torch.float16)
    inp_list, scale_list = ops._views(inp_store, scale_store, table, rws, inp_sizes, scale_sizes, lds)
    out_ptrs, off = [], 0
    for x, r in enumerate(rws):
        if r:
            out_ptrs.append(out_store.data_ptr() + 2 * off)
            off += r * ns[x]
    assert off == bt.out_total

    ptrs, sizes, q = LT.launch_tables(st, rows, bt, inp_store.data_ptr(), scale_store.data_ptr(), out_store.data_ptr())
    live = [x for x, r in enumerate(rws) if r]
    assert ptrs.shape == (6, len(live)) and sizes.dtype == np.uint32 and q.dtype == np.int32
    assert list(ptrs[0]) == [v.data_ptr() for v in inp_list]
    assert list(ptrs[1]) == [b_ptrs[x] for x in live]
    assert list(ptrs[2]) == [0 if v.numel() == 0 else v.data_ptr() for v in scale_list]
    assert list(ptrs[3]) == [sb_ptrs[x] for x in live]
    assert list(ptrs[4]) == out_ptrs
    assert not ptrs[5].any()
    assert sizes.tolist() == [[rws[x], ns[x], widths[x]] for x in live]
    assert q.tolist() == [[qp[x][0], qp[x][1], qp[x][2], int(qp[x][3])] for x in live]


def test_staging_buffer_keeps_every_part_aligned():
    a = np.arange(8, dtype=np.int64).reshape(4, 2)
    b = np.arange(9, dtype=np.uint32).reshape(3, 3)                   # 36 bytes: padded to 40
    c = np.arange(3, dtype=np.int64)
    buf, off = LT.pack_staging([a, b, c])
    assert off == [0, 64, 104] and buf.dtype == np.int64 and buf.nbytes == 128
    raw = buf.view(np.uint8)
    assert np.array_equal(raw[off[1]:off[1] + 36].view(np.uint32), b.reshape(-1))
    assert np.array_equal(raw[off[2]:].view(np.int64), c)


def test_unsupported_activation_format_is_refused():
    with pytest.raises(RuntimeError, match="quant type not supported"):
        LT.static_block([(2, 2, -1, True)], [256], [128], [1], [1])
    with pytest.raises(RuntimeError, match="multiple of 128"):
        LT.static_block([(4, 4, 128, True)], [192], [128], [1], [1])
