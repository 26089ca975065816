"""The permutation entry point that allocates nothing (static device scratch) against the entry point with a caller workspace."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(lib, ids, experts):
    t, k = ids.shape
    r = t * k
    d_ids = torch.from_numpy(ids).to(DEV)
    outs = []
    for static in (False, True):
        dst = torch.full((r,), -7, dtype=torch.int32, device=DEV)
        perm = torch.full((r,), -7, dtype=torch.int64, device=DEV)
        slot = torch.full((r,), -7, dtype=torch.int64, device=DEV)
        recv = torch.full((experts,), -7, dtype=torch.int64, device=DEV)
        s = torch.cuda.current_stream().cuda_stream
        if static:
            rc = lib.mxmoe_build_permutation_static(d_ids.data_ptr(), t, k, experts, dst.data_ptr(), perm.data_ptr(), slot.data_ptr(), recv.data_ptr(), s)
        else:
            ws = torch.empty(lib.mxmoe_permute_workspace_bytes(r, experts), dtype=torch.uint8, device=DEV)
            rc = lib.mxmoe_build_permutation(d_ids.data_ptr(), t, k, experts, dst.data_ptr(), perm.data_ptr(), slot.data_ptr(), recv.data_ptr(), ws.data_ptr(), s)
        assert rc == 0, lib.mxmoe_last_error()
        torch.cuda.synchronize()
        outs.append([x.cpu().numpy() for x in (dst, perm, slot, recv)])
    return outs


def test_static_scratch_permutation_equals_the_workspace_one_on_two_calls(lib):
    rng = np.random.default_rng(31)
    # second call smaller than the first: counters left over from the larger call must not leak into it
    for t, k, e in ((8192, 4, 60), (300, 2, 8)):
        logits = rng.standard_normal((t, e)).astype(np.float32)
        ids, _ = O.route_topk(logits, k)
        ids[rng.integers(0, t, 5), 0] = e + 3                       # a few ids out of range are dropped by both
        ws_out, st_out = _both(lib, ids, e)
        routed = int(ws_out[3].sum())
        assert routed == t * k - 5
        for a, b, name in zip(ws_out, st_out, ("dst_exp_sorted", "perm_indices", "src_slot", "recv")):
            n = len(a) if name == "recv" else routed
            assert np.array_equal(a[:n], b[:n]), f"{name} at T={t}"
        d, p, s_, r = O.permute_by_expert(np.where(ids < e, ids, e), e + 1)
        assert np.array_equal(st_out[0][:routed], d[:routed]) and np.array_equal(st_out[1][:routed], p[:routed])
        assert np.array_equal(st_out[2][:routed], s_[:routed]) and np.array_equal(st_out[3], r[:e])


def test_static_scratch_limit_is_refused_on_the_host(lib):
    cap = lib.mxmoe_static_scratch_bytes()
    assert cap == 1 << 20
    one = (C.c_int64 * 4)()
    a = C.addressof(one)
    rows, e = 256 * 1024, 1024                                      # (1024 blocks + 1) * 1024 experts * 4 bytes > 1 MiB
    assert lib.mxmoe_permute_workspace_bytes(rows, e) > cap
    assert lib.mxmoe_build_permutation_static(a, rows, 1, e, a, a, a, a, None) == 3 and b"static buffer" in lib.mxmoe_last_error()
