"""Offline packers: quantised integers -> the gfx950 operand layouts the kernels read.

Role of the reference's host packers `pack_wxax`, `permute_weight`, `pack_weightonly`, `permute_scale`
(mxmoe/kernels/src/include/quantize.cuh:299-475).  The layouts are this library's own (nothing else reads the
reference's), chosen for 64-lane waves: see csrc/include/mxmoe_tiles.hpp and mxmoe_wo_tiles.hpp.
All functions are pure torch and run on whatever device their input lives on.
"""
from __future__ import annotations

import torch

# element e (0..7) of a dword's eight values sits in nibble (e >> 1) + 4 * (e & 1)
_NIBBLE_OF_ELEM = [(e >> 1) + 4 * (e & 1) for e in range(8)]


def pack_int4_k(q: torch.Tensor) -> torch.Tensor:
    """Signed int4 values [R, K] (in [-8, 7]) -> uint8 [R, K/2]; element 2j in the low nibble of byte j.

    Used for both operands of w4a4 (activations per token, weights per channel), K contiguous as in the
    reference's `pack_wxax` (quantize.cuh:424-475), but with little-endian nibble order.
    """
    assert q.shape[-1] % 2 == 0
    v = q.to(torch.int16) & 0xF
    return (v[..., 0::2] | (v[..., 1::2] << 4)).to(torch.uint8).contiguous()


def unpack_int4_k(p: torch.Tensor) -> torch.Tensor:
    """Inverse of `pack_int4_k` -> int8 [R, K]."""
    lo = (p.to(torch.int16) & 0xF)
    hi = (p.to(torch.int16) >> 4) & 0xF
    v = torch.stack([lo, hi], dim=-1).reshape(*p.shape[:-1], p.shape[-1] * 2)
    return torch.where(v >= 8, v - 16, v).to(torch.int8)


def pack_wxax_fragments(rows: torch.Tensor) -> torch.Tensor:
    """Row-major packed weight bytes [N, KB] (int8 codes, or int4 pairs from `pack_int4_k`; KB a multiple of 64) -> the MFMA
    fragment order the w4a4 / w8a8 tiles load straight into registers: uint8 [ceil(N/32), KB/64, 2, 64, 16] (flattened).

    Block (nb, ks, step) is one 1 KB wave-wide load: lane l = 16-byte k-group (l >> 5) of channel nb*32 + (l & 31), bytes
    ks*64 + (2*step + (l >> 5))*16 .. +16 of that channel's row.  Channels past N are zero rows.
    (The reference's `pack_wxax` / `permute_weight`, quantize.cuh:318-381,424-475, play the same role for ldmatrix.)"""
    r = rows.contiguous().view(torch.uint8)
    n, kb = r.shape
    if kb % 64:
        raise ValueError(f"K must fill whole 64-byte slices of packed codes (128 int4 or 64 int8 values): a row of {kb} bytes does not")
    n32 = (n + 31) // 32
    if n32 * 32 != n:
        r = torch.cat([r, torch.zeros((n32 * 32 - n, kb), dtype=torch.uint8, device=r.device)])
    return r.view(n32, 32, kb // 64, 2, 2, 16).permute(0, 2, 3, 4, 1, 5).contiguous().reshape(-1)


def unpack_wxax_fragments(frag: torch.Tensor, n: int, kb: int) -> torch.Tensor:
    """Inverse of `pack_wxax_fragments` -> uint8 [n, kb]."""
    n32 = (n + 31) // 32
    return frag.view(n32, kb // 64, 2, 2, 32, 16).permute(0, 4, 1, 2, 3, 5).reshape(n32 * 32, kb)[:n].contiguous()


def pack_weight_only(q: torch.Tensor, bits: int) -> torch.Tensor:
    """Unsigned weight codes [N, K] (0 .. 2^bits - 1) -> int32 [N/16, K/128, 64, bits] (flattened to 1-D).

    Lane l of block (nb, kb) carries channel nb*16 + (l & 15), k = kb*128 + (l >> 4)*32 + 0..31.
    bits == 4: dword j holds values 8j..8j+7, value e in nibble (e >> 1) + 4*(e & 1).
    bits == 3: dwords 0..2 hold values 0..23 in the low three bits of their nibbles; bit 3 of nibble p of
    dword d holds bit d of value 24 + e(p).
    bits == 2: dword d holds values 16d..16d+7 in the low two bits of its nibbles and values 16d+8..16d+15 in the high two.
    bits == 8: one byte per value in k order, dword j = values 4j .. 4j+3 (8 dwords per lane).
    """
    assert bits in (2, 3, 4, 8)
    n, k = q.shape
    assert n % 16 == 0 and k % 128 == 0
    v = q.to(torch.int64).reshape(n // 16, 16, k // 128, 4, 32)       # [nb, row, kb, g, e32]
    v = v.permute(0, 2, 3, 1, 4).reshape(n // 16, k // 128, 64, 32)    # lane = g*16 + row
    if bits == 8:
        return v.to(torch.uint8).contiguous().view(torch.int32).reshape(-1).contiguous()
    shifts = torch.tensor([4 * p for p in _NIBBLE_OF_ELEM], dtype=torch.int64, device=q.device)
    if bits == 2:
        pairs = v.reshape(*v.shape[:-1], 2, 2, 8)                      # [.., dword, low / high half of the nibbles, e]
        dw = ((pairs[..., 0, :] | (pairs[..., 1, :] << 2)) << shifts).sum(dim=-1)
        dw = torch.where(dw >= 2**31, dw - 2**32, dw).to(torch.int32)
        return dw.reshape(-1).contiguous()
    ndw = 4 if bits == 4 else 3
    main = v[..., : ndw * 8].reshape(*v.shape[:-1], ndw, 8)
    dw = (main << shifts).sum(dim=-1)                                  # [nb, kb, 64, ndw]
    if bits == 3:
        extra = v[..., 24:32]                                          # values 24..31
        for d in range(3):
            dw[..., d] |= (((extra >> d) & 1) << (shifts + 3)).sum(dim=-1)
    dw = torch.where(dw >= 2**31, dw - 2**32, dw).to(torch.int32)
    return dw.reshape(-1).contiguous()


def pack_weight_only_scales(scale: torch.Tensor, zero: torch.Tensor) -> torch.Tensor:
    """Group scale / zero [N, K/128] fp16 -> fp16 [N/16, K/128, 16, 2] flattened (scale, zero interleaved)."""
    n, g = scale.shape
    assert n % 16 == 0
    sz = torch.stack([scale.to(torch.float16), zero.to(torch.float16)], dim=-1)  # [N, G, 2]
    return sz.reshape(n // 16, 16, g, 2).permute(0, 2, 1, 3).reshape(-1).contiguous()


# ---- int4 values as 6-bit floats (bf6, e3m2): the operand format of the w4a4 tiles on v_mfma_scale_f32_32x32x64_f8f6f4 ----
# Every integer -8 .. 8 is a bf6 number (sign, 3 exponent bits with bias 3, 2 mantissa bits); exponent | mantissa of 0 .. 8:
_BF6_MAGNITUDE = (0, 12, 16, 18, 20, 21, 22, 23, 24)
BF6_FRAGMENT_BYTES = 1536


def bf6_encode(q: torch.Tensor) -> torch.Tensor:
    """Integers -8 .. 8 -> 6-bit bf6 codes (uint8)."""
    if q.numel() and (int(q.min()) < -8 or int(q.max()) > 8):
        raise ValueError("bf6 holds the integers -8 .. 8 exactly, nothing beyond")
    mag = torch.tensor(_BF6_MAGNITUDE, dtype=torch.uint8, device=q.device)
    return mag[q.abs().long()] | ((q < 0).to(torch.uint8) << 5)


def bf6_decode(code: torch.Tensor) -> torch.Tensor:
    """6-bit bf6 codes -> their values as float32 (any code, not only those of integers)."""
    c = code.to(torch.int32)
    e, m = (c >> 2) & 7, c & 3
    val = torch.where(e == 0, m.float() * 0.0625, (1.0 + m.float() * 0.25) * torch.pow(2.0, (e - 3).float()))
    return torch.where((c & 32) != 0, -val, val)


def pack_bf6_fragments(q: torch.Tensor) -> torch.Tensor:
    """[R, K] integers -8 .. 8 (K a multiple of 64; rows are padded with zeros to a multiple of 32) -> uint8
    [ceil(R/32), K/64, 1536] flattened: fragments of 32 rows x 64 k, row block major.  Lane l of a fragment (row l % 32,
    k = 64 ks + 32 (l // 32) + i) holds its 32 codes as 192 bits, value i at bit 6 i; the first 16 bytes of that string lie at byte
    16 l of the fragment, the last 8 at byte 1024 + 8 l.  Both operands of the bf6 tiles use this layout (weights: rows = channels;
    activations: rows = the tokens of one expert, which is what the quantisers write for tag 4)."""
    r, k = q.shape
    if k % 64:
        raise ValueError("K must be a multiple of 64")
    rb = (r + 31) // 32
    if rb * 32 != r:
        q = torch.cat([q, torch.zeros((rb * 32 - r, k), dtype=q.dtype, device=q.device)])
    c = bf6_encode(q).view(rb, 32, k // 64, 2, 32).permute(0, 2, 3, 1, 4).contiguous()      # [row block, k step, k half, row, value]
    bits = (c.unsqueeze(-1) >> torch.arange(6, device=q.device, dtype=torch.uint8)) & 1      # value i -> bits 6 i .. 6 i + 5
    bits = bits.reshape(rb, k // 64, 64, 24, 8)                                               # lane = row + 32 * k half; 192 bits = 24 bytes
    by = (bits << torch.arange(8, device=q.device, dtype=torch.uint8)).sum(-1).to(torch.uint8)
    return torch.cat([by[..., :16].reshape(rb, k // 64, 1024), by[..., 16:].reshape(rb, k // 64, 512)], dim=-1).reshape(-1).contiguous()


def unpack_bf6_fragments(frag: torch.Tensor, r: int, k: int) -> torch.Tensor:
    """Inverse of `pack_bf6_fragments` -> float32 [r, k] (the values the codes stand for)."""
    rb = (r + 31) // 32
    f = frag.view(torch.uint8).reshape(rb, k // 64, 1536)
    by = torch.cat([f[..., :1024].reshape(rb, k // 64, 64, 16), f[..., 1024:].reshape(rb, k // 64, 64, 8)], dim=-1)   # [rb, ks, lane, 24]
    bits = ((by.unsqueeze(-1) >> torch.arange(8, device=frag.device, dtype=torch.uint8)) & 1).reshape(rb, k // 64, 64, 32, 6)
    code = (bits << torch.arange(6, device=frag.device, dtype=torch.uint8)).sum(-1).to(torch.uint8)                  # [rb, ks, lane, value]
    vals = bf6_decode(code).reshape(rb, k // 64, 2, 32, 32).permute(0, 3, 1, 2, 4).reshape(rb * 32, k)
    return vals[:r].contiguous()
