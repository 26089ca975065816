"""Host checks of the packed layouts: a numpy model of the kernels' in-register unpack must invert the packers."""
import numpy as np
import torch

from mxmoe_amd import pack

NIB = [(e >> 1) + 4 * (e & 1) for e in range(8)]


def _cvt8(d, mask_bits):
    """Model of SkinnyWoTile::cvt8: (d & LO), (d & HI), then the same on d >> 8 -> 8 values in k order."""
    d = d.astype(np.uint64)
    lo = (1 << mask_bits) - 1
    out = np.zeros(d.shape + (8,), dtype=np.int64)
    for half, src in enumerate((d, d >> 8)):
        out[..., 4 * half + 0] = src & lo                    # low half of (x & MASK_LO)
        out[..., 4 * half + 1] = (src >> 16) & lo            # high half
        out[..., 4 * half + 2] = (src >> 4) & lo             # low half of (x & MASK_HI), weight 16 folded by the 64.0 magic
        out[..., 4 * half + 3] = (src >> 20) & lo
    return out


def _unpack_model(dw, bits):
    dw = dw.astype(np.int64) & 0xFFFFFFFF
    if bits == 4:
        return np.concatenate([_cvt8(dw[..., j], 4) for j in range(4)], axis=-1)
    if bits == 2:  # out[2d] = cvt8(d), out[2d + 1] = cvt8(d >> 2), two-bit masks
        return np.concatenate([_cvt8(dw[..., d] >> sh, 2) for d in range(2) for sh in (0, 2)], axis=-1)
    t = ((dw[..., 0] >> 3) & 0x11111111) | ((dw[..., 1] >> 2) & 0x22222222) | ((dw[..., 2] >> 1) & 0x44444444)
    return np.concatenate([_cvt8(dw[..., j], 3) for j in range(3)] + [_cvt8(t, 3)], axis=-1)


def test_int4_k_pack_roundtrip_and_nibble_order():
    q = torch.randint(-8, 8, (7, 64), dtype=torch.int8)
    p = pack.pack_int4_k(q)
    assert p.shape == (7, 32) and p.dtype == torch.uint8
    assert torch.equal(pack.unpack_int4_k(p), q)
    one = torch.zeros(1, 4, dtype=torch.int8)
    one[0, 0], one[0, 1] = 3, -2
    assert pack.pack_int4_k(one)[0, 0].item() == (3 | (14 << 4))       # element 0 low nibble, element 1 high nibble
    # kernel-side widening: (x << 4) & 0xF0 and x & 0xF0 as int8 equal 16 * value
    b = p.numpy().astype(np.uint8)
    even = ((b.astype(np.uint16) << 4) & 0xF0).astype(np.uint8).view(np.int8)
    odd = (b & 0xF0).view(np.int8)
    assert np.array_equal(even, 16 * q.numpy()[:, 0::2]) and np.array_equal(odd, 16 * q.numpy()[:, 1::2])


def test_weight_only_pack_matches_kernel_unpack_model():
    for bits in (4, 3, 2):
        n, k = 48, 384
        codes = torch.randint(0, 1 << bits, (n, k), dtype=torch.uint8)
        dw = pack.pack_weight_only(codes, bits).numpy().reshape(n // 16, k // 128, 64, bits)
        vals = _unpack_model(dw, bits)                               # [nb, kb, lane, 32]
        for nb in range(n // 16):
            for kb in range(k // 128):
                for lane in (0, 1, 15, 16, 37, 63):
                    row = nb * 16 + (lane & 15)
                    k0 = kb * 128 + (lane >> 4) * 32
                    assert np.array_equal(vals[nb, kb, lane], codes[row, k0:k0 + 32].numpy())
        assert dw.size * 4 == n * k * bits // 8                         # exactly `bits` bits per weight


def test_weight_only_scale_table_layout():
    n, g = 32, 3
    s = torch.arange(n * g, dtype=torch.float16).reshape(n, g)
    z = -s
    t = pack.pack_weight_only_scales(s, z).reshape(n // 16, g, 16, 2)
    assert t[1, 2, 5, 0] == s[16 + 5, 2] and t[1, 2, 5, 1] == z[16 + 5, 2]


def test_wxax_fragment_order_round_trip_and_lane_map():
    """Weights of the w4a4 / w8a8 tiles: block (nb, ks, step) is one 1 KB wave load, lane l = k-group l >> 5 of channel l & 31."""
    torch.manual_seed(0)
    n, kb = 70, 192                                               # 70 channels (padded to 96), 3 slices of 64 bytes
    rows = torch.randint(0, 256, (n, kb), dtype=torch.uint8)
    frag = pack.pack_wxax_fragments(rows)
    assert frag.numel() == 96 * kb
    assert torch.equal(pack.unpack_wxax_fragments(frag, n, kb), rows)
    f = frag.view(3, 3, 2, 64, 16)
    for (nb, ks, step, lane) in [(0, 0, 0, 0), (1, 2, 1, 37), (2, 1, 0, 63), (2, 0, 1, 5)]:
        ch, kg = nb * 32 + (lane & 31), lane >> 5
        want = rows[ch, ks * 64 + (2 * step + kg) * 16: ks * 64 + (2 * step + kg) * 16 + 16] if ch < n else torch.zeros(16, dtype=torch.uint8)
        assert torch.equal(f[nb, ks, step, lane], want)


def test_bf6_codes_and_fragment_layout():
    """bf6 (e3m2, bias 3) codes of the integers -8 .. 8 decode to themselves, and the fragment buffer holds, for lane l of fragment
    (row block, k step), row l % 32 and k = 64 * step + 32 * (l // 32) + i as value i at bit 6 i of 24 bytes split 16 + 8; rows are
    padded to whole blocks of 32; unpacking returns the values."""
    import torch

    from mxmoe_amd import pack

    q = torch.arange(-8, 9, dtype=torch.int8)
    codes = pack.bf6_encode(q)
    assert codes.tolist() == [56, 55, 54, 53, 52, 50, 48, 44, 0, 12, 16, 18, 20, 21, 22, 23, 24]
    assert pack.bf6_decode(codes).tolist() == [float(v) for v in range(-8, 9)]
    assert pack.bf6_decode(torch.tensor([1, 2, 3, 4, 63], dtype=torch.uint8)).tolist() == [0.0625, 0.125, 0.1875, 0.25, -28.0]  # subnormals, largest
    x = torch.randint(-8, 9, (50, 192), dtype=torch.int8, generator=torch.Generator().manual_seed(4))
    buf = pack.pack_bf6_fragments(x)
    f = buf.numpy().reshape(2, 3, pack.BF6_FRAGMENT_BYTES)
    for rb in range(2):
        for ks in range(3):
            for lane in (0, 1, 17, 31, 32, 47, 63):
                raw = bytes(f[rb, ks, 16 * lane:16 * lane + 16]) + bytes(f[rb, ks, 1024 + 8 * lane:1024 + 8 * lane + 8])
                v = int.from_bytes(raw, "little")
                vals = pack.bf6_decode(torch.tensor([(v >> (6 * i)) & 63 for i in range(32)], dtype=torch.uint8)).to(torch.int8)
                row, k0 = 32 * rb + lane % 32, 64 * ks + 32 * (lane // 32)
                assert torch.equal(vals, x[row, k0:k0 + 32] if row < 50 else torch.zeros(32, dtype=torch.int8))
    assert torch.equal(pack.unpack_bf6_fragments(buf, 50, 192), x.float())
    import pytest

    with pytest.raises(ValueError):
        pack.bf6_encode(torch.tensor([9], dtype=torch.int8))
    with pytest.raises(ValueError):
        pack.pack_bf6_fragments(torch.zeros(32, 96, dtype=torch.int8))
