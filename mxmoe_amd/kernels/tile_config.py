"""Tile descriptors of the gfx950 kernels, with the reference's class and field names.

`TileConfig` / `QConfig` / `NO_QUANT` keep the fields (and therefore the dataclass `repr`, which is the key of the
kernel-profile table) of mxmoe/kernels/tile_config.py:122-286.  What changes is the meaning the hardware gives them:
WM x WN x WK counts 64-lane wavefronts (always 4 per workgroup here), MMA names an MFMA instruction, STAGE is the number of
LDS ring slots of the DMA pipeline (3 for the MFMA tiles; for the few-token weight-only tiles 2 names the 12-deep register ring with 4 k blocks per pass and 4 the few-register shape), and the candidate lists are those compiled for gfx950.
"""
from __future__ import annotations

import dataclasses
import re


def get_gpu_info() -> dict:
    """Replaces the pycuda / pynvml probe (tile_config.py:3-30): arch, compute-unit count, LDS per CU, clock."""
    import torch

    if not torch.cuda.is_available():
        return {"cc": "gfx950", "sm_count": 256, "frequency": (2400, 2400), "max_shared_memory_per_mp": 160 * 1024}
    p = torch.cuda.get_device_properties(0)
    arch = getattr(p, "gcnArchName", "gfx950").split(":")[0]
    clk = int(getattr(p, "clock_rate", 2400000) // 1000)
    return {"cc": arch, "sm_count": p.multi_processor_count, "frequency": (clk, clk), "max_shared_memory_per_mp": 160 * 1024}


TYPE_TO_BITS = {
    **dict.fromkeys(["half", "bfloat16"], 16),
    **dict.fromkeys(["float", "int32_t"], 32),
    **dict.fromkeys(["int8_t", "uint8_t"], 8),
    **dict.fromkeys(["int4_t", "uint4_t"], 4),
    **dict.fromkeys(["int3_t", "uint3_t"], 3),
    **dict.fromkeys(["int2_t", "uint2_t"], 2),
}

# weight-only formats: bits x group size (128, or -1 = one scale per channel) x symmetric / asymmetric (tile_config.py:40-59 lists
# 8 / 4 / 2 bits with both group sizes; 3 bits is this library's addition)
WEIGHT_ONLY_QCFG = [f"w{w}a16_g{g}_{s}" for w in (8, 4, 3, 2) for g in (128, -1) for s in ("sym", "asym")]

# The reference's "_accfp16" names (fp16 accumulators in its mma instructions, tile_config.py:41,50-56): the matrix instructions of
# gfx950 accumulate fp16 products in fp32 only, so these names are accepted and built as the fp32-accumulating tiles of the base format.
ACCFP16_ALIASES = {"fp16_accfp16": "fp16", **{f"{q}_accfp16": q for q in WEIGHT_ONLY_QCFG}}

SUPPORTED_QCFG = [
    "fp16",
    "bf16",  # bfloat16 operands and outputs, fp32 accumulation (tile_config.py:42): the QParams of fp16, told apart by the kernel (a variant)
    "w8a8_g-1_sym",
    "w8a8_g-1_sym_E4M3",  # fp8 (OCP e4m3) codes on both sides, fp32 accumulation (tile_config.py:45)
    "w4a4_g-1_sym",
    "w4a4_g128_sym",
    *WEIGHT_ONLY_QCFG,
    *ACCFP16_ALIASES,
]

# (M, N, K) of one MFMA instruction
MMA_SHAPE = {
    "MFMA_F32_32x32x16_F16": (32, 32, 16),
    "MFMA_F32_32x32x16_BF16": (32, 32, 16),
    "MFMA_I32_32x32x32_I8": (32, 32, 32),
    "MFMA_I32_32x32x32_I8_FROM_I4": (32, 32, 32),  # int4 operands widened to int8 (16*v) in registers
    "MFMA_F32_16x16x32_F16": (16, 16, 32),
    # int4 values held as 6-bit floats (bf6, e3m2: every integer -8 .. 8 is one) on v_mfma_scale_f32_32x32x64_f8f6f4 with unit
    # scales: the fp32 accumulators are the exact integer sums, at twice the int8 instruction's rate
    "MFMA_F32_32x32x64_BF6_FROM_I4": (32, 32, 64),
    "MFMA_F32_32x32x16_FP8": (32, 32, 16),
}
MMA_TO_ACC_TYPE = {"MFMA_F32_32x32x16_F16": "float", "MFMA_F32_32x32x16_BF16": "float", "MFMA_I32_32x32x32_I8": "int32_t", "MFMA_I32_32x32x32_I8_FROM_I4": "int32_t", "MFMA_F32_16x16x32_F16": "float",
                   "MFMA_F32_32x32x64_BF6_FROM_I4": "float", "MFMA_F32_32x32x16_FP8": "float"}
MMA_TO_INP_TYPE = {"MFMA_F32_32x32x16_F16": "half", "MFMA_F32_32x32x16_BF16": "bfloat16", "MFMA_I32_32x32x32_I8": "int8_t", "MFMA_I32_32x32x32_I8_FROM_I4": "int4_t", "MFMA_F32_16x16x32_F16": "half",
                   "MFMA_F32_32x32x64_BF6_FROM_I4": "int4_t", "MFMA_F32_32x32x16_FP8": "fp8e4m3"}
BF6_MMA = "MFMA_F32_32x32x64_BF6_FROM_I4"

QCFG_TO_MMA = {
    "fp16": "MFMA_F32_32x32x16_F16",
    "bf16": "MFMA_F32_32x32x16_BF16",
    "w8a8_g-1_sym": "MFMA_I32_32x32x32_I8",
    "w8a8_g-1_sym_E4M3": "MFMA_F32_32x32x16_FP8",
    "w4a4_g-1_sym": "MFMA_I32_32x32x32_I8_FROM_I4",
    "w4a4_g128_sym": "MFMA_I32_32x32x32_I8_FROM_I4",
    **{q: "MFMA_F32_16x16x32_F16" for q in WEIGHT_ONLY_QCFG},
}
QCFG_TO_MMA.update({alias: QCFG_TO_MMA[base] for alias, base in ACCFP16_ALIASES.items()})


@dataclasses.dataclass
class QConfigBase:
    T_PACK: str = "half"
    QBITS: int = 16
    GSIZE: int = -1
    SYM: bool = True
    PACK_DIM: str = "PackDim::K"
    USE_FP: bool = False
    T_SCALE: str = "half"

    def bytes_per_scale_zp(self):
        raise NotImplementedError

    def pack_num(self):
        return 16 // self.QBITS

    def qtype(self):
        if self.QBITS >= 16:
            return None
        return f"{'int' if self.SYM else 'uint'}{self.QBITS}_t"


@dataclasses.dataclass
class NO_QUANT(QConfigBase):
    def to_str(self):
        return "NO_QUANT"

    def bytes_per_scale_zp(self):
        return 0


@dataclasses.dataclass
class QConfig(QConfigBase):
    def to_str(self):
        return f"QConfig<{self.T_PACK}, {'true' if self.SYM else 'false'}, {self.QBITS}, {self.GSIZE}, {self.PACK_DIM}, {'true' if self.USE_FP else 'false'}, {self.T_SCALE}>"

    def bytes_per_scale_zp(self):
        return TYPE_TO_BITS[self.T_SCALE] // 8 * (1 if self.SYM else 2)


QCFG_W8A8 = QConfig(QBITS=8, GSIZE=-1, SYM=True, PACK_DIM="PackDim::K")
QCFG_W8A8_E4M3 = QConfig(QBITS=8, GSIZE=-1, SYM=True, PACK_DIM="PackDim::K", USE_FP=True)
QCFG_W4A4 = QConfig(QBITS=4, GSIZE=-1, SYM=True, PACK_DIM="PackDim::K")
QCFG_W4A4_G128 = QConfig(QBITS=4, GSIZE=128, SYM=True, PACK_DIM="PackDim::K")

CFG_TEMPLATE = "TileConfig<{BM},{BN},{BK},{WM},{WN},{WK},{STAGE},{SPLITK},{MMA},{QCFGA},{QCFGB}>"


@dataclasses.dataclass
class TileConfig:
    BM: int = 64
    BN: int = 64
    BK: int = 64
    WM: int = 2
    WN: int = 2
    WK: int = 1
    STAGE: int = 2
    SPLITK: int = -1
    MMA: str = "MFMA_F32_32x32x16_F16"
    QCFGA: QConfigBase = dataclasses.field(default_factory=NO_QUANT)
    QCFGB: QConfigBase = dataclasses.field(default_factory=NO_QUANT)

    def to_str(self):
        return CFG_TEMPLATE.format(BM=self.BM, BN=self.BN, BK=self.BK, WM=self.WM, WN=self.WN, WK=self.WK, STAGE=self.STAGE, SPLITK=self.SPLITK,
                                   MMA=self.MMA, QCFGA=self.QCFGA.to_str(), QCFGB=self.QCFGB.to_str())

    def __hash__(self):
        return hash(self.to_str())

    def __eq__(self, other):
        return isinstance(other, TileConfig) and dataclasses.asdict(self) == dataclasses.asdict(other)

    @property
    def num_warps(self):
        """Wavefronts per workgroup (the reference's warps per CTA); fused branches must agree (compose_kernel.py:69-71)."""
        return self.WM * self.WN * self.WK

    def warp_tile_mnk(self):
        return self.BM // self.WM, self.BN // self.WN, self.BK // self.WK

    def w_bits(self):
        return self.QCFGB.QBITS

    def a_bits(self):
        return self.QCFGA.QBITS

    def acc_type(self):
        return MMA_TO_ACC_TYPE[self.MMA]

    def is_a_quant(self):
        return not isinstance(self.QCFGA, NO_QUANT)

    def is_b_quant(self):
        return not isinstance(self.QCFGB, NO_QUANT)

    def set_qcfg(self, qcfg: "TileConfig") -> "TileConfig":
        self.QCFGA, self.QCFGB = qcfg.QCFGA, qcfg.QCFGB
        return self

    def is_weight_only(self) -> bool:
        return self.MMA == "MFMA_F32_16x16x32_F16"

    def is_skinny(self) -> bool:
        return self.is_weight_only() and self.BM in (16, 32)

    def is_bf6(self) -> bool:
        """int4 operands handed over as bf6 fragments (both activations and weights; the quantisers write them, tag 4)."""
        return self.MMA == BF6_MMA

    def is_group_wa(self) -> bool:
        """Both operands int4 with a scale per 128-wide K group (w4a4_g128_sym)."""
        return self.MMA == "MFMA_I32_32x32x32_I8_FROM_I4" and getattr(self.QCFGA, "GSIZE", -1) == 128

    def smem_bytes_scale(self):
        return 0  # scales are read straight from global memory in the epilogue / per group

    def smem_bytes_tile(self):
        """LDS bytes of the tile as compiled (csrc/include/mxmoe_tiles.hpp, mxmoe_wo_tiles.hpp)."""
        if self.is_skinny():  # per-wave partial sums of the final reduction + (scale, zero) patches of one pass (4 k blocks, or 2)
            kp = 2 if self.STAGE == 4 or self.BM == 32 else 4
            return 4 * (self.BN // 16) * (64 * 16 * (self.BM // 16) + kp * 64)
        if self.is_weight_only():
            return 2 * self.BM * 256  # two stages of BM activation rows x one 128-wide k block
        if self.is_group_wa():
            return self.STAGE * self.BM * 64
        if self.is_bf6():  # four stages of the tile's token fragments (1536 bytes per 32 rows, rounded up to 1 KB pieces), or the epilogue patch
            return max(4 * (-(-(self.BM // 32 * 1536) // 1024) * 1024), 4 * 32 * (64 * 2 + 16))
        if self.MMA != "MFMA_F32_32x32x16_F16":  # activations only: 3 stages of BM x 64 B, or the epilogue patch if larger
            return max(self.STAGE * self.BM * 64, 4 * min(self.BM, 64) * (64 * 2 + 8))
        return self.STAGE * (self.BM + self.BN) * 64

    def cpp_type(self) -> str:
        """The C++ tile type this descriptor instantiates."""
        if self.is_skinny():
            if self.BM == 32:  # two blocks of 16 tokens against every unpacked weight: 2 k blocks per pass, 8 (8-bit: 4) packed blocks in flight
                return f"SkinnyWoTile<{self.QCFGB.QBITS}, {self.BN}, 2, {4 if self.QCFGB.QBITS == 8 else 8}, 2, 2>"
            # STAGE 4: the few-register shape (2 k blocks per pass, 4 packed blocks in flight per wave, compiled for 3 waves per SIMD)
            return f"SkinnyWoTile<{self.QCFGB.QBITS}, {self.BN}, 2, 4, 3>" if self.STAGE == 4 else f"SkinnyWoTile<{self.QCFGB.QBITS}, {self.BN}>"
        if self.is_weight_only():
            return f"WoMfmaTile<{self.QCFGB.QBITS}, {self.BM}, {self.BN}>"
        if self.is_bf6():
            return f"Bf6Tile<{self.BM}>"
        op = {"MFMA_F32_32x32x16_F16": "Op::F16", "MFMA_F32_32x32x16_BF16": "Op::BF16", "MFMA_I32_32x32x32_I8": "Op::I8", "MFMA_I32_32x32x32_I8_FROM_I4": "Op::I4", "MFMA_F32_32x32x16_FP8": "Op::F8"}[self.MMA]
        if self.is_group_wa():
            return f"WxAxGTile<{self.BM}>"
        if op not in ("Op::F16", "Op::BF16"):
            return f"WxAxTile<{op}, {self.BM}, {self.BN}>"
        return f"MfmaTile<{op}, {self.BM}, {self.BN}, {self.WM}, {self.WN}>"

    def validate(self) -> None:
        if self.num_warps != 4:
            raise ValueError(f"{self!r}: gfx950 tiles use 4 wavefronts per workgroup")
        if self.is_weight_only():
            if self.BK != 128 or not ((self.BM in (16, 32) and self.BN % 64 == 0 and (self.WM, self.WN) == (1, 4)) or (self.BM, self.BN, self.WM, self.WN) in ((128, 128, 2, 2), (128, 256, 1, 4))):
                raise ValueError(f"{self!r}: weight-only tiles are 16 or 32 x (64k) x 128 (1 x 4 waves), 128 x 128 x 128 (2 x 2 waves) or 128 x 256 x 128 (1 x 4 waves)")
            return
        if self.is_bf6():
            if (self.BN, self.BK, self.WM, self.WN, self.WK, self.STAGE) != (256, 64, 1, 4, 1, 4) or self.BM not in (32, 64, 128):
                raise ValueError(f"{self!r}: bf6 tiles are BM x 256 x 64 with 1 x 4 waves and 4 stages, BM in 32 / 64 / 128")
            return
        k_elems = {"MFMA_F32_32x32x16_F16": 32, "MFMA_F32_32x32x16_BF16": 32, "MFMA_I32_32x32x32_I8": 64, "MFMA_I32_32x32x32_I8_FROM_I4": 128, "MFMA_F32_32x32x16_FP8": 64}[self.MMA]
        if self.BK != k_elems or self.STAGE != 3 or self.WK != 1 or (self.BM // self.WM) % 32 or (self.BN // self.WN) % 32:
            raise ValueError(f"{self!r}: unsupported shape for {self.MMA} (BK must be {k_elems}, STAGE 3, wave tile a multiple of 32x32)")
        if self.is_group_wa() and self.BM not in (32, 64):
            raise ValueError(f"{self!r}: group-quantised int4 tiles are 32 x 256 or 64 x 256 (two sets of accumulators)")
        if self.MMA not in ("MFMA_F32_32x32x16_F16", "MFMA_F32_32x32x16_BF16") and ((self.WM, self.WN) != (1, 4) or self.BN != 256 or self.BM not in (32, 64, 128)):
            raise ValueError(f"{self!r}: integer tiles are BM x 256 with 1 x 4 waves (each wave streams its own 64 weight channels), BM in 32 / 64 / 128")


def get_info_from_qcfg_str(qcfg: str):
    """'w4a4_g-1_sym' -> (w_bits, a_bits, gsize, sym)   (tile_config.py:288-294)."""
    if qcfg.startswith("fp16") or qcfg == "bf16":
        return 16, 16, -1, True
    s = qcfg.split("_")
    wbits = int(s[0].split("a")[0].split("w")[1])
    abits = int(s[0].split("a")[1])
    return wbits, abits, int(s[1].split("g")[1]), s[2] == "sym"


def build_qcfgb_from_str(qcfg: str) -> QConfig:
    w, _a, g, sym = get_info_from_qcfg_str(qcfg)
    return QConfig(QBITS=w, GSIZE=g, SYM=sym, PACK_DIM="PackDim::MN")


QCFG_MAP = {
    "fp16": TileConfig(),
    "bf16": TileConfig(),
    "w8a8_g-1_sym": TileConfig(QCFGA=QCFG_W8A8, QCFGB=QCFG_W8A8),
    "w8a8_g-1_sym_E4M3": TileConfig(QCFGA=QCFG_W8A8_E4M3, QCFGB=QCFG_W8A8_E4M3),
    "w4a4_g-1_sym": TileConfig(QCFGA=QCFG_W4A4, QCFGB=QCFG_W4A4),
    "w4a4_g128_sym": TileConfig(QCFGA=QCFG_W4A4_G128, QCFGB=QCFG_W4A4_G128),
    **{k: TileConfig(QCFGB=build_qcfgb_from_str(k)) for k in WEIGHT_ONLY_QCFG},
}
QCFG_MAP.update({alias: QCFG_MAP[base] for alias, base in ACCFP16_ALIASES.items()})


def _with_q(t: TileConfig, qcfg: str) -> TileConfig:
    return dataclasses.replace(t, QCFGA=QCFG_MAP[qcfg].QCFGA, QCFGB=QCFG_MAP[qcfg].QCFGB)


def get_possible_tile_list(arch: str, qcfg: str) -> list:
    """Candidate tiles per qcfg (hand-curated like tile_config.py:330-610, for gfx950)."""
    if not str(arch).startswith("gfx95"):
        raise ValueError(f"no tile list for arch {arch!r}: this library targets gfx950")
    mma = QCFG_TO_MMA[qcfg]
    if mma == "MFMA_F32_16x16x32_F16":
        skinny = [_with_q(TileConfig(BM=16, BN=bn, BK=128, WM=1, WN=4, WK=1, STAGE=2, MMA=mma), qcfg) for bn in (128, 64)]
        skinny.append(_with_q(TileConfig(BM=32, BN=128, BK=128, WM=1, WN=4, WK=1, STAGE=2, MMA=mma), qcfg))  # experts with 17 .. 32 (.. 64) tokens
        if QCFG_MAP[qcfg].QCFGB.QBITS != 8:  # the few-register shape, for kernels made of few-token tiles alone (three workgroups per CU)
            skinny.append(_with_q(TileConfig(BM=16, BN=128, BK=128, WM=1, WN=4, WK=1, STAGE=4, MMA=mma), qcfg))
        # (8-bit weights: the ring of packed blocks is twice as large, which leaves room for the 2 x 2 shape's accumulators only)
        shapes = ((128, 2, 2),) if QCFG_MAP[qcfg].QCFGB.QBITS == 8 else ((128, 2, 2), (256, 1, 4))
        big = [_with_q(TileConfig(BM=128, BN=bn, BK=128, WM=wm, WN=wn, WK=1, STAGE=2, MMA=mma), qcfg) for bn, wm, wn in shapes]
        return skinny + big
    bk = {"MFMA_F32_32x32x16_F16": 32, "MFMA_F32_32x32x16_BF16": 32, "MFMA_I32_32x32x32_I8": 64, "MFMA_I32_32x32x32_I8_FROM_I4": 128, "MFMA_F32_32x32x16_FP8": 64}[mma]
    if mma in ("MFMA_F32_32x32x16_F16", "MFMA_F32_32x32x16_BF16"):
        shapes = [(128, 256, 2, 2), (64, 256, 1, 4), (32, 256, 1, 4), (128, 128, 2, 2), (256, 128, 2, 2)]
    elif qcfg == "w4a4_g128_sym":
        shapes = [(64, 256, 1, 4), (32, 256, 1, 4)]
    else:
        shapes = [(128, 256, 1, 4), (64, 256, 1, 4), (32, 256, 1, 4)]
    tiles = [_with_q(TileConfig(BM=bm, BN=bn, BK=bk, WM=wm, WN=wn, WK=1, STAGE=3, MMA=mma), qcfg) for bm, bn, wm, wn in shapes]
    if qcfg == "w4a4_g-1_sym":  # the same shapes on the 6-bit float path (operands as bf6 fragments): never mixed with the tiles above in one kernel
        tiles += [_with_q(TileConfig(BM=bm, BN=256, BK=64, WM=1, WN=4, WK=1, STAGE=4, MMA=BF6_MMA), qcfg) for bm in (128, 64, 32)]
    return tiles


_FIELD = re.compile(r"(BM|BN|BK|WM|WN|WK|STAGE|SPLITK)=(-?\d+)")


def parse_tile_repr(text: str, qcfg: str | None = None) -> list:
    """Parse TileConfig reprs (the form `bits_solver.export_qconfig` writes: `{layer: repr(tuple_of_TileConfig)}`,
    bits_solver.py:30,67-69) back into TileConfig objects."""
    out = []
    for chunk in text.split("TileConfig(")[1:]:
        vals = {k: int(v) for k, v in _FIELD.findall(chunk.split("QCFGA")[0])}
        mma = re.search(r"MMA='([^']+)'", chunk)
        t = TileConfig(MMA=mma.group(1) if mma else TileConfig().MMA, **vals)
        out.append(_with_q(t, qcfg) if qcfg else t)
    return out


def tile_from_dict(d: dict, qcfg: str) -> TileConfig:
    """`{BM, BN, BK, WM, WN, WK, STAGE, SPLITK, MMA}` -> TileConfig carrying the qcfg's QCFGA / QCFGB."""
    keys = ("BM", "BN", "BK", "WM", "WN", "WK", "STAGE", "SPLITK", "MMA")
    t = TileConfig(**{k: d[k] for k in keys if k in d})
    if "MMA" not in d:
        t.MMA = QCFG_TO_MMA[qcfg]
    return _with_q(t, qcfg)


def load_tile_configs(obj: dict, qcfgs) -> dict:
    """Accept both tile_config JSON forms: `{qcfg: [tile dicts or repr strings]}` (what run_mxmoe_gg.py:101-106 expects)
    and `{layer: repr(tuple_of_TileConfig)}` (what the ILP writes); returns `{qcfg: [TileConfig]}`."""
    qcfgs = sorted(qcfgs)
    out = {}
    if all(k in QCFG_MAP for k in obj):
        for q, items in obj.items():
            tiles = []
            for it in items if isinstance(items, list) else [items]:
                tiles += [tile_from_dict(it, q)] if isinstance(it, dict) else parse_tile_repr(it, q)
            out[q] = tiles
        return out
    for _layer, text in obj.items():  # repr form: one tile per qcfg in sorted-qcfg order
        tiles = parse_tile_repr(text)
        for q, t in zip(qcfgs, tiles):
            out.setdefault(q, []).append(_with_q(t, q))
    return out
