"""Template generator: qcfg set x tile candidates -> fused gfx950 kernels, compiled with hipcc into one shared library.

Same entry point as the reference (mxmoe/kernels/compose_kernel.py:79-572):
    TemplateGenerator(arch, qcfgs, KernelType.Fused, tile_configs).generate_source_code()
emits `generated/hz_fused_decl.hpp` + one `generated/hz_fused_<i>.hip` per fusion-compatible combination of one tile per
qcfg (cartesian product filtered by equal wavefront count, compose_kernel.py:87-108), each registering
`groupgemm_hz_fused_<i>`.  `build()` then replaces the reference's cmake + ninja step (run_mxmoe_gg.py:109-111).

`KernelType.Sequential` / `MultiStream` (the reference's ablation launchers, kernel_sketch.py:148-406) emit one
single-format kernel per qcfg; the launch policy for them lives in mxmoe_amd.harness.
"""
from __future__ import annotations

import argparse
import enum
import os
from collections import OrderedDict
from itertools import product
from pathlib import Path

from .. import build as _build
from .kernel_sketch import ABI_TU, KERNEL_DECLARATION_TEMPLATE, KERNEL_DEFINITION_TEMPLATE
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


BRANCH_CONDITION_MAP = {"fp16": "(a_bits == 16 && w_bits == 16)", **{k: _gen_condition(k) for k in SUPPORTED_QCFG if k != "fp16"}}

GEN_DIR = Path(__file__).resolve().parent.parent / "csrc" / "generated"


def is_fusion_compatible(tile_cfgs) -> bool:
    return all(tile_cfgs[0].num_warps == c.num_warps for c in tile_cfgs)


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
            for t in tiles:
                t.validate()
        if self.kernel_type == KernelType.Fused:
            combos = [c for c in product(*per_q.values()) if is_fusion_compatible(c)]
            return [OrderedDict(zip(per_q.keys(), c)) for c in combos]
        # one single-format kernel per (qcfg, tile)
        return [OrderedDict([(q, t)]) for q, tiles in per_q.items() for t in tiles]

    def get_smem_size(self, tile_cfg_dict) -> tuple:
        return max(t.smem_bytes_tile() for t in tile_cfg_dict.values()), max(t.smem_bytes_scale() for t in tile_cfg_dict.values())

    def cvt_qcfg_str_to_condition(self, qcfg: str) -> str:
        assert qcfg in self.qcfgs, f"Invalid qcfg: {qcfg}"
        return BRANCH_CONDITION_MAP[qcfg]

    def build_single_kernel(self, tile_cfg: OrderedDict, kname: str):
        tiles = ", ".join(t.cpp_type() for t in tile_cfg.values())
        comment = "; ".join(f"{q} if {BRANCH_CONDITION_MAP[q]} -> {t.to_str()}" for q, t in tile_cfg.items())
        defn = KERNEL_DEFINITION_TEMPLATE.substitute(KernelName=kname, Tiles=tiles, Comment=comment)
        decl = f"//   {kname}: " + ", ".join(f"[{q}: ({t.BM},{t.BN},{t.BK}) ({t.WM},{t.WN},{t.WK}) {t.STAGE}]" for q, t in tile_cfg.items())
        return decl, defn

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

    def build(self, out: str | os.PathLike | None = None) -> Path:
        """hipcc the generated translation units into one shared library exporting the C-ABI."""
        out = Path(out) if out else self.out_dir / f"libmxmoe_{self.kernel_type}.so"
        return _build.hipcc_build(self.files, out)


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
