"""Kernel-profile table: producer (on gfx950) and consumer.

The table is the input of the reference's bit-width / tile allocator: `{qcfg: {slot: {repr(TileConfig): {"first_iter_cost",
"inc", "stderr"}}}}` in milliseconds (the reference keeps one for sm_89 in perf/performance_table.json; its producer is not
part of the reference).  The consumer `get_runtime_cost` restates mxmoe/quant/bits_solver.py:518-542:
`cost[expert][block][strategy][tile combo] = table[qcfg][slot][repr(tile)]["inc"] * num_tiles(shape, tile)`.

Meaning of the fields as regenerated here (the reference documents none):
  * a *tile wave* is `cus` tiles (256: one tile per compute unit);
  * a single-format, single-tile kernel is timed on problems of 1, 2, 3, 4, 6 and 8 tile waves at reduction depth
    K = 1024 * slot (slots "1".."4"), median of the harness' timed launches each;
  * `first_iter_cost` = time of the one-wave problem, `inc` = least-squares slope in ms per added tile wave,
    `stderr` = standard error of that slope.
Compute-bound tiles (w4a4, w8a8, fp16) grow M (weights N = 8 tile columns); skinny weight-only tiles keep M = 16 rows and grow N, the
shape they exist for (every added tile streams new weights from HBM).
"""
from __future__ import annotations

import argparse
import itertools
import json
import math
from dataclasses import dataclass
from pathlib import Path

from .kernels.compose_kernel import KernelType, TemplateGenerator, is_fusion_compatible
from .kernels.tile_config import QCFG_MAP, TileConfig, get_info_from_qcfg_str, get_possible_tile_list

WAVES = (1, 2, 3, 4, 6, 8)
SLOTS = ("1", "2", "3", "4")


@dataclass
class ProblemShape:
    """bits_solver.py:104-110."""
    M: int
    N: int
    K: int

    def num_tiles(self, tile: TileConfig) -> int:
        return ((self.M + tile.BM - 1) // tile.BM) * ((self.N + tile.BN - 1) // tile.BN)


def slot_of(qcfg: str) -> str:
    """The slot the allocator reads: "1" for weight-only formats, "3" for weight-activation formats (bits_solver.py:533-537)."""
    return "1" if "a16" in qcfg else "3"


def table_key(qcfg: str) -> str:
    """bits_solver.py:531-532: w2a16_g128_asym is looked up under its fp16-accumulate variant."""
    return "w2a16_g128_asym_accfp16" if qcfg == "w2a16_g128_asym" else qcfg


def get_runtime_cost(workloads, strategy_list, performance_table: dict, tile_cfgs: dict | None = None, arch: str = "gfx950"):
    """Runtime cost of every (expert, linear block, strategy, tile combination)  (bits_solver.py:518-542).

    workloads: [expert][block] -> ProblemShape; strategy_list: qcfg strings; tile_cfgs: optional {qcfg: [TileConfig]} (default: the
    arch's candidate list, the role of the reference's hand-picked `get_best_tile_configs`).
    Returns (tile combinations, cost[e][block][strategy][combination])."""
    if tile_cfgs is not None:
        per_q = {q: list(tile_cfgs[q]) for q in strategy_list}
    else:
        per_q = {q: [t.set_qcfg(QCFG_MAP[q]) for t in get_possible_tile_list(arch, q)] for q in strategy_list}
    combos = [c for c in itertools.product(*per_q.values()) if is_fusion_compatible(c)]
    cost = []
    for exp in workloads:
        cost.append([])
        for w in exp:
            cost[-1].append([])
            for j, qcfg in enumerate(strategy_list):
                perf = performance_table[table_key(qcfg)][slot_of(qcfg)]
                cost[-1][-1].append([perf[repr(c[j])]["inc"] * w.num_tiles(c[j]) for c in combos])
    return combos, cost


def linear_fit(xs, ys):
    """Least-squares line through (xs, ys): (intercept, slope, standard error of the slope)."""
    n = len(xs)
    mx, my = sum(xs) / n, sum(ys) / n
    sxx = sum((x - mx) ** 2 for x in xs)
    slope = sum((x - mx) * (y - my) for x, y in zip(xs, ys)) / sxx
    icpt = my - slope * mx
    rss = sum((y - icpt - slope * x) ** 2 for x, y in zip(xs, ys))
    return icpt, slope, math.sqrt(rss / max(n - 2, 1) / sxx)


def sweep_entry(tile: TileConfig, qcfg: str, k: int, waves: int, cus: int = 256) -> dict:
    """One-problem workload entry of `waves` tile waves for `tile`."""
    w_bits, a_bits, gsize, sym = get_info_from_qcfg_str(qcfg)
    if tile.is_skinny():
        m, n = tile.BM, tile.BN * cus * waves
    else:
        m, n = tile.BM * (cus // 8) * waves, tile.BN * 8
    return {"shape": [m, n, k], "w_bits": w_bits, "a_bits": a_bits, "gsize": gsize, "sym": sym}


def build_qcfg_lib(qcfg: str, arch: str = "gfx950", rebuild: bool = False):
    """One library of single-tile kernels (one per candidate tile of `qcfg`); returns (library path, tiles in kernel order).
    An existing library is reused unless `rebuild`, so it can be compiled on a machine without a GPU beforehand."""
    from .kernels.compose_kernel import GEN_DIR

    gen = TemplateGenerator(arch, [qcfg], KernelType.Fused, out_dir=GEN_DIR / f"perf_{qcfg}")  # one qcfg: one single-tile kernel per candidate
    gen.generate_source_code()
    so = gen.out_dir / f"libmxmoe_{gen.kernel_type}.so"
    if rebuild or not so.exists():
        gen.build(so)
    return so, [next(iter(c.values())) for c in gen.combos]


def profile_qcfg(qcfg: str, arch: str = "gfx950", slots=SLOTS, waves=WAVES, rebuild: bool = False, verbose: bool = True) -> dict:
    """Time the wave sweep of every candidate tile of `qcfg`; returns {slot: {repr(tile): fit}}."""
    import torch

    from . import _lib, harness

    so, tiles = build_qcfg_lib(qcfg, arch, rebuild)
    lib = _lib.load(so)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    res = {s: {} for s in slots}
    for s in slots:
        k = 1024 * int(s)
        for kid, tile in enumerate(tiles):
            ts = []
            for w in waves:
                prob = harness.make_problem(sweep_entry(tile, qcfg, k, w, cus), None)
                launch = harness._launch_of([prob], lib, kid)
                ts.append(harness.bench_func(launch.run, warmup=5, iters=20)["median"])
                del prob, launch
            _, slope, err = linear_fit(list(waves), ts)
            res[s][repr(tile)] = {"first_iter_cost": round(ts[0], 5), "inc": round(slope, 5), "stderr": err}
            if verbose:
                print(f"{qcfg} slot {s} ({tile.BM},{tile.BN},{tile.BK}) ({tile.WM},{tile.WN},{tile.WK}): first {ts[0]:.4f} ms, inc {slope:.5f} ms/wave, stderr {err:.2e}", flush=True)
        torch.cuda.empty_cache()
    return res


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Regenerate the kernel-profile table on this GPU")
    ap.add_argument("--qcfgs", nargs="+", default=["w4a4_g-1_sym", "w8a8_g-1_sym", "w4a16_g128_asym", "w3a16_g128_asym", "w2a16_g128_asym", "w4a4_g128_sym", "fp16"])
    ap.add_argument("--slots", nargs="+", default=list(SLOTS))
    ap.add_argument("--out", default="perf/performance_table.json")
    ap.add_argument("--build-only", action="store_true", help="compile the single-tile kernel libraries and stop (needs no GPU)")
    ap.add_argument("--rebuild", action="store_true")
    a = ap.parse_args(argv)
    if a.build_only:
        for q in a.qcfgs:
            print(build_qcfg_lib(q, rebuild=True)[0])
        return 0
    out = Path(a.out)
    table = json.loads(out.read_text()) if out.exists() else {}
    for q in a.qcfgs:
        table[q] = profile_qcfg(q, slots=a.slots, rebuild=a.rebuild)
        out.parent.mkdir(parents=True, exist_ok=True)
        out.write_text(json.dumps(table, indent=1))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
