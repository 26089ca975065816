"""Quantise + pack one weight matrix [N, K] for a format; the result is what `Bs[p]` / `scale_b[p]` point to."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import pack
from .quant import quant_minmax


@dataclass
class PackedWeight:
    data: torch.Tensor            # packed weights in the kernel's layout
    scale: torch.Tensor | None    # per-channel scales [N] (w-a) or group (scale, zero) table (weight-only)
    qparams: tuple                # (a_bits, w_bits, gsize, sym)
    n: int
    k: int
    q: torch.Tensor | None = None  # integer codes [N, K] (kept only when asked; tests)

    @property
    def nbytes(self) -> int:
        return self.data.numel() * self.data.element_size() + (0 if self.scale is None else self.scale.numel() * self.scale.element_size())


def quantize_and_pack(w: torch.Tensor, qparams, keep_codes: bool = False, bf6: bool = False, fp8: bool = False) -> PackedWeight:
    """RTN-quantise `w` [N, K] fp16 for `(a_bits, w_bits, gsize, sym)` and pack it.

    fp16: kept as is.  w8a8 / w4a4: per-channel symmetric codes (int8 / packed nibbles, K contiguous) re-ordered into MFMA
    fragment blocks (`pack.pack_wxax_fragments`), fp16 scale [N].
    With `fp8`, w8a8 weights are fp8 e4m3 codes (same layout as int8) for the kernels whose w8a8 tiles run the fp8 instruction.
    With `bf6`, w4a4 weights become bf6 fragments (`pack.pack_bf6_fragments`) for the kernels whose w4a4 tiles run on the 6-bit
    float matrix path; every other format is unaffected.
    w8a16 / w4a16 / w3a16 / w2a16, group 128 or per channel (-1): unsigned codes in the wave-interleaved layout with a (scale, zero) table; symmetric
    variants are stored offset-binary with zero = -2^(b-1) * scale (exact).
    """
    a_bits, w_bits, gsize, sym = qparams
    n, k = w.shape
    if w_bits >= 16:
        return PackedWeight(w.contiguous(), None, tuple(qparams), n, k)
    if fp8 and (a_bits, w_bits, gsize) == (8, 8, -1):
        # w8a8 on the fp8 instruction (the reference's w8a8_g-1_sym_E4M3): per-channel e4m3 codes in the int8 tiles' fragment order
        from .quant import quant_e4m3

        codes, scale = quant_e4m3(w)
        return PackedWeight(pack.pack_wxax_fragments(codes), scale.reshape(n).contiguous(), tuple(qparams), n, k, codes if keep_codes else None)
    q, scale, zp = quant_minmax(w, w_bits, gsize, sym)
    return pack_codes(q, scale, zp, qparams, n, k, keep_codes, bf6)


def pack_codes(q: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor, qparams, n: int, k: int, keep_codes: bool = False, bf6: bool = False) -> PackedWeight:
    """Pack integer codes `q` [N, K] with their fp16 `scale` / `zp` (one per channel, or per channel and group; value = q * scale + zp)
    into the kernels' layouts.  Symmetric codes are signed, asymmetric ones 0 .. 2^bits - 1."""
    a_bits, w_bits, gsize, sym = qparams
    if a_bits < 16 and gsize == 128:
        # w4a4_g128_sym: codes as for w4a4, one scale per channel and 128-wide K group, stored group-major [K/128, N] so that a
        # tile reads the scales of its channels for one group as one contiguous run
        assert sym and w_bits == 4 and a_bits == 4 and k % 128 == 0, "group-quantised w-a format: w4a4_g128_sym"
        qi = q.reshape(n, k).to(torch.int8)
        data = pack.pack_wxax_fragments(pack.pack_int4_k(qi))
        return PackedWeight(data, scale.reshape(n, k // 128).t().contiguous(), tuple(qparams), n, k, qi if keep_codes else None)
    if a_bits < 16:
        assert gsize == -1 and sym, "w-a formats are per-channel symmetric"
        qi = q.to(torch.int8)
        if bf6 and w_bits == 4:  # for the tiles on the 6-bit float path (kernels "..._b6"): the same codes as bf6 fragments
            return PackedWeight(pack.pack_bf6_fragments(qi.reshape(n, k)), scale.reshape(n).contiguous(), tuple(qparams), n, k, qi if keep_codes else None)
        data = pack.pack_wxax_fragments(qi if w_bits == 8 else pack.pack_int4_k(qi))
        return PackedWeight(data, scale.reshape(n).contiguous(), tuple(qparams), n, k, qi if keep_codes else None)
    # weight-only: one (scale, zero) pair per channel and 128-wide K group.  Per-channel formats (group size -1) repeat the channel's
    # pair for every group: the tiles apply the pair group by group either way.
    assert gsize in (128, -1) and k % 128 == 0, "weight-only kernels take group size 128 or -1 (per channel), K a multiple of 128"
    g = k // 128
    scale = scale.reshape(n, -1).expand(n, g) if gsize == -1 else scale.reshape(n, g)
    zp = zp.reshape(n, -1).expand(n, g) if gsize == -1 else zp.reshape(n, g)
    codes = q.reshape(n, k)
    if sym:
        off = 1 << (w_bits - 1)
        codes = codes + off
        zp = (-off * scale).to(scale.dtype)
    codes = codes.to(torch.uint8)
    return PackedWeight(pack.pack_weight_only(codes, w_bits), pack.pack_weight_only_scales(scale.contiguous(), zp.contiguous()), tuple(qparams), n, k,
                        codes if keep_codes else None)
