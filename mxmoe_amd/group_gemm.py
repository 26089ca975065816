"""Python face of the fused GroupGEMM launch: device pointer tables + one C-ABI call per launch.

Host-side counterpart of `moe_mxmoe_share_fused` (mxmoe/kernels/src/ref_bind.cu:312-431): it builds the same
five pointer arrays, the problem sizes and the QParams list, but once, into one device buffer that is reused by
every launch (the reference re-allocates and re-copies them on every call, ref_bind.cu:395-404,426-428).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from .weights import PackedWeight  # noqa: F401  (re-export for callers)


class GroupGemmLaunch:
    """A prepared problem list: `run()` is a single allocation-free, sync-free kernel launch."""

    def __init__(self, As, Bs, scale_a, scale_b, Cs, sizes, qparams, kernel_id: int = -1, acc=None, lib=None):
        self.lib = lib or _lib.load()
        p = len(As)
        assert len(Bs) == len(Cs) == len(sizes) == len(qparams) == p
        self.count = p
        self.kernel_id = kernel_id
        self._keep = (As, Bs, scale_a, scale_b, Cs, acc)  # keep the tensors alive
        dev = Cs[0].device if p else torch.device("cuda")

        def ptrs(ts):
            return [0 if t is None or t.numel() == 0 else t.data_ptr() for t in ts]

        cols = [ptrs(As), ptrs(Bs), ptrs(scale_a or [None] * p), ptrs(scale_b or [None] * p), ptrs(Cs), ptrs(acc or [None] * p)]
        table = torch.tensor(cols, dtype=torch.int64).reshape(6, p)
        self.h_sizes = (_lib.Dim3 * max(p, 1))(*[_lib.Dim3(int(m), int(n), int(k)) for (m, n, k) in sizes])
        self.h_q = (_lib.QParams * max(p, 1))(*[_lib.QParams(int(a), int(w), int(g), 1 if s else 0) for (a, w, g, s) in qparams])
        sz = torch.tensor([[int(m), int(n), int(k)] for (m, n, k) in sizes], dtype=torch.int32).reshape(p, 3)
        self.d_table = table.to(dev)
        self.d_sizes = sz.to(dev)
        self.has_acc = acc is not None
        self.sizes = [tuple(int(v) for v in s) for s in sizes]
        self.ops = sum(2 * m * n * k for (m, n, k) in self.sizes)

    def _ptr(self, row: int) -> int:
        return self.d_table.data_ptr() + row * self.count * 8

    def run(self, stream=None) -> None:
        if self.count == 0:
            return
        s = stream if stream is not None else torch.cuda.current_stream().cuda_stream
        rc = self.lib.mxmoe_group_gemm(
            self.kernel_id, self._ptr(0), self._ptr(1), self._ptr(2), self._ptr(3), self._ptr(4), self._ptr(4),
            None, None, None, None, self.d_sizes.data_ptr(), self.h_sizes, None, self.h_q, self.count,
            self._ptr(5) if self.has_acc else None, s,
        )
        _lib.check(self.lib, rc)

    def plan(self):
        """(kernel id, branch per problem, total tiles) the launcher would use."""
        br = (C.c_int32 * max(self.count, 1))()
        tiles = C.c_int32(0)
        rc = self.lib.mxmoe_group_gemm_plan(self.kernel_id, self.h_sizes, self.h_q, self.count, br, C.byref(tiles))
        if rc < 1000:
            _lib.check(self.lib, rc or 1)
        return rc - 1000, list(br)[: self.count], tiles.value
