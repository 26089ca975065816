"""int4 values as bf6 (e3m2) fragments for the 6-bit float matrix path (diagnostic kernel `mxmoe_bf6_gemm_probe`).

Every integer -8 .. 8 is a bf6 number: sign bit, 3 exponent bits (bias 3), 2 mantissa bits.  A fragment is what one
v_mfma_scale_f32_32x32x64_f8f6f4 takes from a wave: 32 rows x 64 k, lane l holding row l % 32 and k = 32 * (l // 32) + 0..31 as
32 codes = 192 bits (value i at bit 6 i); its first 16 bytes lie at byte 16 l of the fragment, its last 8 bytes at 1024 + 8 l.
Fragments are stored k step major: offset(row block, k step) = (k step * rows / 32 + row block) * 1536."""
from __future__ import annotations

import torch

_MAGNITUDE = (0, 12, 16, 18, 20, 21, 22, 23, 24)  # exponent | mantissa of 0 .. 8
FRAGMENT_BYTES = 1536


def encode(q: torch.Tensor) -> torch.Tensor:
    """Integers -8 .. 8 -> 6-bit bf6 codes (uint8)."""
    if q.numel() and (int(q.min()) < -8 or int(q.max()) > 8):
        raise ValueError("bf6 holds the integers -8 .. 8 exactly, nothing beyond")
    mag = torch.tensor(_MAGNITUDE, dtype=torch.uint8, device=q.device)
    return mag[q.abs().long()] | ((q < 0).to(torch.uint8) << 5)


def decode(code: torch.Tensor) -> torch.Tensor:
    """6-bit bf6 codes -> their values as float32 (any code, not only those of integers)."""
    c = code.to(torch.int32)
    e, m = (c >> 2) & 7, c & 3
    val = torch.where(e == 0, m.float() * 0.0625, (1.0 + m.float() * 0.25) * torch.pow(2.0, (e - 3).float()))
    return torch.where((c & 32) != 0, -val, val)


def pack_fragments(q: torch.Tensor) -> torch.Tensor:
    """[R, K] integers -8 .. 8 (R a multiple of 32, K of 64) -> the fragment-ordered uint8 buffer described above."""
    r, k = q.shape
    if r % 32 or k % 64:
        raise ValueError("rows must be a multiple of 32 and K of 64")
    c = encode(q).view(r // 32, 32, k // 64, 2, 32).permute(2, 0, 3, 1, 4).contiguous()  # [k step, row block, k half, row, value]
    bits = (c.unsqueeze(-1) >> torch.arange(6, device=q.device, dtype=torch.uint8)) & 1      # value i -> bits 6 i .. 6 i + 5
    bits = bits.reshape(k // 64, r // 32, 64, 24, 8)                                          # lane = row + 32 * k half; 192 bits = 24 bytes
    by = (bits << torch.arange(8, device=q.device, dtype=torch.uint8)).sum(-1).to(torch.uint8)
    return torch.cat([by[..., :16].reshape(k // 64, r // 32, 1024), by[..., 16:].reshape(k // 64, r // 32, 512)], dim=-1).reshape(-1).contiguous()
