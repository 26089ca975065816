"""Template generator: qcfg set x tile candidates -> fused gfx950 kernels, compiled with hipcc into one shared library.

Same entry point as the reference (mxmoe/kernels/compose_kernel.py:79-572):
    TemplateGenerator(arch, qcfgs, KernelType.Fused, tile_configs).generate_source_code()
emits `generated/hz_fused_decl.hpp` + one `generated/hz_fused_<i>.hip` per fusion-compatible combination of one tile per
qcfg (cartesian product filtered by equal wavefront count, compose_kernel.py:87-108), each registering
`groupgemm_hz_fused_<i>`.  `build()` then replaces the reference's cmake + ninja step (run_mxmoe_gg.py:109-111).

A qcfg's entry in `tile_configs` may also be a tuple of TileConfig (a *shape set*): the kernel then carries every shape of
the set as a branch of that format and its host launcher picks the shapes per problem from the row count (whole tiles of the
cheapest shape per row, the remainder with the shape that covers it most cheaply).  The kernels of the default library
(`default_kernel_specs`) are such sets; `emit_default_library` writes their translation unit, which the package build compiles.

`KernelType.Sequential` / `MultiStream` (the reference's ablation launchers, kernel_sketch.py:148-406) emit the same
combinations registered with the sequential / multi-stream launch policy of the C++ host launcher: one launch per run of
consecutive problems of equal format, on the caller's stream or on side streams.
"""
from __future__ import annotations

import argparse
import enum
import os
from collections import OrderedDict
from itertools import product
from pathlib import Path

from .. import build as _build
from .kernel_sketch import ABI_TU, DEFAULT_ORDER_TEMPLATE, KERNEL_DECLARATION_TEMPLATE, KERNEL_DEFERRED_TEMPLATE, KERNEL_DEFINITION_TEMPLATE
from .tile_config import QCFG_MAP, SUPPORTED_QCFG, TileConfig, get_gpu_info, get_info_from_qcfg_str, get_possible_tile_list  # noqa: F401


class KernelType(str, enum.Enum):
    Fused = "hz_fused"
    Sequential = "seq_launch"
    MultiStream = "ms_launch"

    def __str__(self):
        return self.value


def _gen_condition(qcfg: str) -> str:
    w, a, g, sym = get_info_from_qcfg_str(qcfg)
    return f"(a_bits == {a} && w_bits == {w} && gsize == {g} && sym == {'true' if sym else 'false'})"


BRANCH_CONDITION_MAP = {"fp16": "(a_bits == 16 && w_bits == 16)", "bf16": "(a_bits == 16 && w_bits == 16)",
                        **{k: _gen_condition(k) for k in SUPPORTED_QCFG if k not in ("fp16", "bf16")}}

GEN_DIR = Path(__file__).resolve().parent.parent / "csrc" / "generated"


POLICY = {"hz_fused": "Policy::Fused", "seq_launch": "Policy::Sequential", "ms_launch": "Policy::MultiStream"}


def _flat(items):
    """Tiles of a combination, shape sets expanded."""
    out = []
    for it in items:
        out += list(it) if isinstance(it, (tuple, list)) else [it]
    return out


def is_fusion_compatible(tile_cfgs) -> bool:
    tiles = _flat(tile_cfgs)
    return all(tiles[0].num_warps == c.num_warps for c in tiles)


class TemplateGenerator:
    def __init__(self, arch: str, qcfgs, kernel_type: KernelType = KernelType.Fused, tile_configs: dict | None = None, out_dir: str | os.PathLike | None = None):
        for q in qcfgs:
            if q not in SUPPORTED_QCFG:
                raise ValueError(f"Unsupported qcfg: {q}")
        self.arch = arch
        self.qcfgs = sorted(qcfgs)
        self.kernel_type = KernelType(kernel_type)
        self.tile_configs = tile_configs
        self.out_dir = Path(out_dir) if out_dir else GEN_DIR
        self.kernel_names: list[str] = []

    def get_tile_configs(self) -> list:
        if self.tile_configs is not None:
            per_q = OrderedDict((q, list(self.tile_configs[q])) for q in self.qcfgs)
        else:
            per_q = OrderedDict((q, get_possible_tile_list(self.arch, q)) for q in self.qcfgs)
        for tiles in per_q.values():
            for t in _flat(tiles):
                t.validate()
        combos = [c for c in product(*per_q.values()) if is_fusion_compatible(c)]
        return [OrderedDict(zip(per_q.keys(), c)) for c in combos]

    def get_smem_size(self, tile_cfg_dict) -> tuple:
        tiles = _flat(tile_cfg_dict.values())
        return max(t.smem_bytes_tile() for t in tiles), max(t.smem_bytes_scale() for t in tiles)

    def cvt_qcfg_str_to_condition(self, qcfg: str) -> str:
        assert qcfg in self.qcfgs, f"Invalid qcfg: {qcfg}"
        return BRANCH_CONDITION_MAP[qcfg]

    def build_single_kernel(self, tile_cfg: OrderedDict, kname: str):
        return build_kernel_source(tile_cfg, kname, self.kernel_type)

    def generate_source_code(self) -> list:
        combos = self.get_tile_configs()
        self.out_dir.mkdir(parents=True, exist_ok=True)
        for old in self.out_dir.glob(f"{self.kernel_type}_*"):
            old.unlink()
        decls, files = [], []
        self.kernel_names = []
        for i, combo in enumerate(combos):
            kname = f"groupgemm_{self.kernel_type}_{i}"
            decl, defn = self.build_single_kernel(combo, kname)
            decls.append(decl)
            path = self.out_dir / f"{self.kernel_type}_{i}.hip"
            path.write_text(defn)
            files.append(path)
            self.kernel_names.append(kname)
        (self.out_dir / f"{self.kernel_type}_decl.hpp").write_text(KERNEL_DECLARATION_TEMPLATE.substitute(Signatures="\n".join(decls)))
        abi = self.out_dir / f"{self.kernel_type}_abi.hip"
        abi.write_text(ABI_TU)
        files.append(abi)
        self.files = files
        self.combos = combos
        print(f"Generated {len(combos)} kernels for `{self.kernel_type}` {self.qcfgs}")
        return files

    def library_path(self) -> Path:
        """Where `build()` puts the library of this generator's kernels: the file name carries a digest of the kernel set, so two
        format or tile sets never share a name (a process that loads both would otherwise get the first one back from the loader
        the second time: shared libraries are cached by name)."""
        import hashlib

        text = ";".join(f"{self.kernel_type}_{i}:" + ",".join(f"{q}={t.to_str()}" for q, item in combo.items() for t in _flat([item]))
                        for i, combo in enumerate(self.get_tile_configs()))
        return self.out_dir / f"libmxmoe_{self.kernel_type}_{hashlib.sha1(text.encode()).hexdigest()[:10]}.so"

    def build(self, out: str | os.PathLike | None = None) -> Path:
        """hipcc the generated translation units into one shared library exporting the C-ABI."""
        if out is None:
            out = self.library_path()
            for old in self.out_dir.glob(f"libmxmoe_{self.kernel_type}*.so"):  # libraries of earlier kernel sets in this directory
                if old != out:
                    old.unlink()
        return _build.hipcc_build(self.files, Path(out))


def build_kernel_source(tile_cfg, kname: str, kernel_type: KernelType = KernelType.Fused, deferred: bool = False, max_rows_hint: int = 0):
    """(declaration comment, translation unit) of one kernel; `tile_cfg` maps qcfg -> TileConfig or tuple of TileConfig.
    `deferred`: the unit defines `register_<kname>()` instead of registering from a static initialiser.  `max_rows_hint`: the kernel
    is meant for problems of at most that many rows (the launcher's automatic choice prefers it when no problem has more)."""
    pairs = [(q, t) for q, item in tile_cfg.items() for t in _flat([item])]
    tiles = ", ".join(t.cpp_type() for _, t in pairs)
    comment = "; ".join(f"{q} if {BRANCH_CONDITION_MAP[q]} -> {t.to_str()}" for q, t in pairs)
    defn = (KERNEL_DEFERRED_TEMPLATE if deferred else KERNEL_DEFINITION_TEMPLATE).substitute(KernelName=kname, Tiles=tiles, Comment=comment, Policy=POLICY[str(kernel_type)],
                                                                                                  Hint=f", {max_rows_hint}" if max_rows_hint else "")
    decl = f"//   {kname}: " + ", ".join(f"[{q}: ({t.BM},{t.BN},{t.BK}) ({t.WM},{t.WN},{t.WK}) {t.STAGE}]" for q, t in pairs)
    return decl, defn


def _pick(arch: str, qcfg: str, *shapes, bf6: bool = False, few_registers: bool = False):
    """Candidate tiles of `qcfg` with the given (BM, BN) shapes, in that order (`bf6`: the tiles on the 6-bit float path;
    `few_registers`: the few-token weight-only tiles in their few-register shape)."""
    by_shape = {(t.BM, t.BN): t for t in get_possible_tile_list(arch, qcfg) if t.is_bf6() == bf6 and (t.is_skinny() and t.STAGE == 4) == few_registers}
    return tuple(by_shape[s] for s in shapes)


def default_kernel_specs(arch: str = "gfx950"):
    """The kernels of libmxmoe_amd.so: (function name, kernel type, {qcfg: shape set}) in registry order."""
    w4, w8 = "w4a4_g-1_sym", "w8a8_g-1_sym"
    wo = OrderedDict((f"w{b}a16_g128_asym", _pick(arch, f"w{b}a16_g128_asym", (16, 128), (32, 128))) for b in (4, 3, 2))
    wo_big = OrderedDict((f"w{b}a16_g128_asym", _pick(arch, f"w{b}a16_g128_asym", (128, 256))) for b in (4, 3, 2))
    wo_all = OrderedDict((q, wo[q] + wo_big[q]) for q in wo)
    everything = OrderedDict([(w4, _pick(arch, w4, (128, 256), (32, 256))), (w8, _pick(arch, w8, (128, 256), (32, 256))),
                              ("fp16", _pick(arch, "fp16", (128, 256), (32, 256))), *wo_all.items(), ("w4a4_g128_sym", _pick(arch, "w4a4_g128_sym", (64, 256))),
                              ("w8a16_g128_asym", _pick(arch, "w8a16_g128_asym", (16, 128), (32, 128), (128, 128)))])
    everything_b6 = OrderedDict(everything)
    everything_b6[w4] = _pick(arch, w4, (128, 256), (32, 256), bf6=True)
    everything_e4m3 = OrderedDict(("w8a8_g-1_sym_E4M3" if q == w8 else q, _pick(arch, "w8a8_g-1_sym_E4M3", (128, 256), (32, 256)) if q == w8 else t) for q, t in everything.items())
    return [
        ("groupgemm_hz_fused_wxax", KernelType.Fused, OrderedDict([(w4, _pick(arch, w4, (128, 256), (64, 256), (32, 256))), (w8, _pick(arch, w8, (128, 256), (64, 256), (32, 256)))])),
        ("groupgemm_hz_fused_fp16", KernelType.Fused, OrderedDict([("fp16", _pick(arch, "fp16", (128, 256), (64, 256), (32, 256)))])),
        ("groupgemm_hz_fused_wo", KernelType.Fused, wo_all),
        ("groupgemm_hz_fused_wxax_g128", KernelType.Fused, OrderedDict([("w4a4_g128_sym", _pick(arch, "w4a4_g128_sym", (64, 256), (32, 256)))])),
        # every format in one launch (layers that mix weight-only, w-a and fp16 blocks), and the same kernel behind the two ablation policies
        ("groupgemm_hz_fused_all", KernelType.Fused, everything),
        ("groupgemm_seq_launch_all", KernelType.Sequential, everything),
        ("groupgemm_ms_launch_all", KernelType.MultiStream, everything),
        # the same two kernels with w4a4 on the 6-bit float path: both operands of a w4a4 problem are bf6 fragments (the quantisers'
        # tag 4, pack.pack_bf6_fragments).  Registered last: a caller that does not ask for them by name never gets them.
        # 8-bit weight-only formats in a kernel of their own (their tiles hold twice the packed registers of the 4-bit ones; a kernel
        # runs at the occupancy of its largest branch)
        # the few-token tiles of the 4 / 3 / 2-bit weight-only formats alone: without the many-token tiles' registers three workgroups
        # share a CU instead of two, which is what these latency-bound weight streams gain from (decode-sized batches)
        ("groupgemm_hz_fused_wo_skinny", KernelType.Fused,
         OrderedDict((f"w{b}a16_g128_asym", _pick(arch, f"w{b}a16_g128_asym", (16, 128), few_registers=True)) for b in (4, 3, 2))),
        ("groupgemm_hz_fused_wo8", KernelType.Fused, OrderedDict([("w8a16_g128_asym", _pick(arch, "w8a16_g128_asym", (16, 128), (32, 128), (128, 128)))])),
        # w8a8 in fp8 (e4m3 codes on both sides), next to w4a4
        ("groupgemm_hz_fused_wxax_e4m3", KernelType.Fused, OrderedDict([(w4, _pick(arch, w4, (128, 256), (64, 256), (32, 256))),
                                                                         ("w8a8_g-1_sym_E4M3", _pick(arch, "w8a8_g-1_sym_E4M3", (128, 256), (64, 256), (32, 256)))])),
        ("groupgemm_hz_fused_wxax_b6", KernelType.Fused, OrderedDict([(w4, _pick(arch, w4, (128, 256), (64, 256), (32, 256), bf6=True)), (w8, _pick(arch, w8, (128, 256), (64, 256), (32, 256)))])),
        ("groupgemm_hz_fused_all_b6", KernelType.Fused, everything_b6),
        ("groupgemm_hz_fused_all_e4m3", KernelType.Fused, everything_e4m3),
        # bfloat16 operands and outputs (the reference's "bf16"): the QParams of fp16 problems, so by name only
        ("groupgemm_hz_fused_bf16", KernelType.Fused, OrderedDict([("bf16", _pick(arch, "bf16", (128, 256), (64, 256), (32, 256)))])),
    ]


# default kernels meant for problems of few rows only
MAX_ROWS_HINT = {"groupgemm_hz_fused_wo_skinny": 64}


def emit_default_library(out_dir: str | os.PathLike | None = None, arch: str = "gfx950") -> list:
    """Write the translation units that register the default kernels, one per kernel (they compile in parallel), and return
    their paths in registry order.  Static initialisers of different translation units run in link order, which is the order of
    this list, so every unit registers through one ordered table instead: unit i only fills slot i, and the last step of
    library start-up (the unit written last) registers the slots in order."""
    out_dir = Path(out_dir) if out_dir else GEN_DIR
    out_dir.mkdir(parents=True, exist_ok=True)
    specs = default_kernel_specs(arch)
    paths, keep = [], set()
    for kname, ktype, tile_cfg in specs:
        for t in _flat(tile_cfg.values()):
            t.validate()
        if not is_fusion_compatible(list(tile_cfg.values())):
            raise ValueError(f"{kname}: branches disagree on the wavefront count")
        _decl, defn = build_kernel_source(tile_cfg, kname, ktype, deferred=True, max_rows_hint=MAX_ROWS_HINT.get(kname, 0))
        path = out_dir / f"default_{kname}.hip"
        if not path.exists() or path.read_text() != defn:
            path.write_text(defn)
        paths.append(path)
        keep.add(path.name)
    order = out_dir / "default_order.hip"
    text = DEFAULT_ORDER_TEMPLATE.substitute(Decls="\n".join(f"int register_{k}();" for k, _t, _c in specs),
                                             Calls="\n".join(f"    register_{k}();" for k, _t, _c in specs))
    if not order.exists() or order.read_text() != text:
        order.write_text(text)
    keep.add(order.name)
    for old in out_dir.glob("default_*.hip"):
        if old.name not in keep:
            old.unlink()
    return paths + [order]


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description="Compose kernel")
    p.add_argument("--type", type=str, default="Fused", choices=["Fused", "Sequential", "MultiStream"])
    p.add_argument("--qcfgs", type=str, nargs="+", default=["fp16"])
    p.add_argument("--build", action="store_true")
    a = p.parse_args(argv)
    gen = TemplateGenerator(get_gpu_info()["cc"], a.qcfgs, KernelType[a.type])
    gen.generate_source_code()
    if a.build:
        print(gen.build())
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
