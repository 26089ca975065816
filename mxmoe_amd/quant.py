"""Host-side (torch) RTN quantiser with the reference's exact arithmetic, used to prepare weights offline.

Same operation sequence as `quant_minmax` / `Quantizer` (mxmoe/quant/quant.py:40-109): everything in the
tensor's dtype (fp16 on the path), clamp before round-half-even, float zero point for asymmetric groups.
A zero range maps to scale 1 as in the reference's CUDA quantiser (mxmoe/kernels/src/include/quantize.cuh:258).
"""
from __future__ import annotations

import torch


def quant_minmax(t: torch.Tensor, bits: int, gsize: int, sym: bool, clip=(1.0, 1.0)):
    g = t.shape[-1] if gsize == -1 else gsize
    r = t.reshape(-1, g)
    if sym:
        upper = (1 << (bits - 1)) - 1
        lower = -upper
        scale = r.abs().amax(dim=-1, keepdim=True) / upper
        zp = torch.zeros_like(scale)
    else:
        upper = (1 << bits) - 1
        lower = 0
        gmin, gmax = r.aminmax(dim=-1, keepdim=True)
        gmin = gmin * clip[0]
        gmax = gmax * clip[1]
        scale = (gmax - gmin) / upper
        zp = gmin
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = r.sub(zp).div(scale).clamp(lower, upper).round()
    return q.reshape(t.shape), scale, zp


E4M3_MAX = 448.0


def quant_e4m3(t: torch.Tensor):
    """Per-row fp8 (OCP e4m3) quantisation with the arithmetic of the symmetric integer formats: scale = max|row| / 448 in the
    tensor's dtype (a zero row gets 1), codes = e4m3(clamp(row / scale, +-448)) rounded to nearest even.  Returns (codes uint8 of
    t's shape, scale [rows, 1]).  The format of the reference's w8a8_g-1_sym_E4M3 tiles (mxmoe/kernels/tile_config.py:45,192), whose
    repository holds no quantiser for it."""
    r = t.reshape(-1, t.shape[-1])
    scale = r.abs().amax(dim=-1, keepdim=True) / E4M3_MAX
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = r.div(scale).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float32).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(t.shape), scale


class Quantizer:
    """mxmoe/quant/quant.py:87-109."""

    def __init__(self, bits: int, sym: bool, gsize: int, clip=(1.0, 1.0)):
        self.bits, self.sym, self.gsize, self.clip = bits, sym, gsize, clip

    def quant(self, t):
        if self.bits == 16:
            return t, 1.0, 0.0
        return quant_minmax(t, self.bits, self.gsize, self.sym, self.clip)

    def dequant(self, t, scale, zp):
        if self.bits == 16:
            return t
        g = t.shape[-1] if self.gsize == -1 else self.gsize
        return t.reshape(-1, g).mul(scale).add(zp).reshape(t.shape)

    def fake_quant(self, t):
        if self.bits == 16:
            return t
        return self.dequant(*self.quant(t))

    def __repr__(self):
        return f"Quantizer(bits={self.bits}, sym={self.sym}, gsize={self.gsize}, clip={self.clip})"
