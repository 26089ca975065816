#!/usr/bin/env python3
"""Bench the mixed-precision GroupGEMM kernels of one MoE model on gfx950 — same flags, file names and CSV columns as the
reference entry point (run_mxmoe_gg.py:32-121):

    python run_mxmoe_gg.py [--model {qwen2_moe,qwen2_moe_57b,ds2,mixtral}] [--dataset {wiki2,humaneval-x}]
                           [--qconfig PATH | --qstr STR] [--tile_config PATH] [--bs INT] [--layer INT]

Steps: qcfg set of the qconfig -> workload JSON from the expert-frequency trace (`out/workloads/...`) -> generate the fused
kernels for that qcfg set -> hipcc them into one library (replaces cmake + ninja) -> time every kernel per layer
(`out/bench/{model}-{dataset}-{bs}{suffix}-layer-{i}-{gate_up|down}.csv`, in-process instead of `./build/test bench`).

The reference's traces come from real checkpoints (`calib/gate/{model}/{dataset}/4096/moe-gate.json`).  Without them,
`--synthetic {c1..c5}` writes the trace and qconfig of a seeded synthetic configuration under `out/synthetic/` and uses
those; `--trace PATH` points at any trace file.
"""
import argparse
import json
import os
import sys

from mxmoe_amd.kernels.compose_kernel import KernelType, TemplateGenerator
from mxmoe_amd.kernels.gen_workload import MODEL_ID_TO_LAYERS, MODEL_ID_TO_TRACE_FILE, generate_workload_from_gate_trace
from mxmoe_amd.kernels.tile_config import get_gpu_info, load_tile_configs
from mxmoe_amd.project_config import CUR_DIR


def get_qcfg_list(qcfg_file: str, target_layer: int) -> set:
    """run_mxmoe_gg.py:10-29: the set of "w{w}a{a}_g{g}_{sym|asym}" strings present in the qconfig (one layer or all)."""
    with open(qcfg_file) as f:
        qcfg = json.load(f)
    qcfg.pop("LT", None)
    out = set()
    for layer_idx, v in qcfg.items():
        if target_layer != -1 and int(layer_idx) != target_layer:
            continue
        for _e, qexp in v["experts"].items():
            for _n, lin in qexp.items():
                if lin["w_bits"] >= 16 and lin["a_bits"] >= 16:
                    out.add("fp16")
                else:
                    out.add(f"w{lin['w_bits']}a{lin['a_bits']}_g{lin['w_gsize']}_{'sym' if lin['w_sym'] else 'asym'}")
    return out


def materialise_synthetic(name: str, bs: int | None):
    from mxmoe_amd import synth

    cfg = synth.get_config(name, bs)
    d = f"{CUR_DIR}/out/synthetic"
    os.makedirs(d, exist_ok=True)
    trace, qcfg = f"{d}/{name}-moe-gate.json", f"{d}/{name}-wbits-{name}.json"
    with open(trace, "w") as f:
        json.dump(synth.trace_dict(cfg), f)
    with open(qcfg, "w") as f:
        json.dump(synth.qconfig_dict(cfg), f)
    return cfg, trace, qcfg


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description="Bench workloads for groupgemm kernel.")
    p.add_argument("--model", type=str, default="qwen2_moe", help="Model ID.")
    p.add_argument("--dataset", type=str, default="wiki2", help="Dataset ID.")
    p.add_argument("--qconfig", type=str, default=None, help="Path to the quantization config file.")
    p.add_argument("--tile_config", type=str, default=None, help="Path to the tile config file.")
    p.add_argument("--qstr", type=str, default=None, help="Short string to represent quantization config.")
    p.add_argument("--bs", type=int, default=512, help="Batch size.")
    p.add_argument("--layer", type=int, default=-1, help="Layer index.")
    p.add_argument("--synthetic", type=str, default=None, choices=["c1", "c2", "c3", "c4", "c5"], help="use a seeded synthetic configuration")
    p.add_argument("--trace", type=str, default=None, help="expert-frequency trace file (moe-gate.json)")
    p.add_argument("--mode", type=str, default="bench", choices=["bench", "check"])
    p.add_argument("--max-kernels", type=int, default=0, help="generate at most this many tile combinations (0 = all)")
    p.add_argument("--no-bench", action="store_true", help="stop after the workload file, the generated sources and the library (no GPU needed)")
    args = p.parse_args(argv)

    model_id, dataset, bs, layer = args.model, args.dataset, args.bs, args.layer
    trace = args.trace
    exact = False
    if args.synthetic:
        cfg, trace, synthetic_qcfg = materialise_synthetic(args.synthetic, None if "--bs" not in (argv or sys.argv) else bs)
        # an explicit --qconfig (e.g. one the allocator, mxmoe_amd.bits_solver, wrote for this workload) or --qstr (one format for every
        # block) wins over the configuration's own seeded formats
        args.qconfig = args.qconfig or (None if args.qstr is not None else synthetic_qcfg)
        model_id, dataset, bs, layer, exact = cfg.model, "synthetic", cfg.tokens, 0, True

    if args.qconfig is not None:
        qcfg_list = get_qcfg_list(args.qconfig, layer)
        workload_suffix = "-" + args.qconfig.split("wbits")[1].split(".json")[0] + ".json" if args.qconfig != "" else ".json"
    elif args.qstr is not None:
        qcfg_list = [args.qstr]
        workload_suffix = f"-{args.qstr}.json"
    else:
        qcfg_list = ["fp16"]
        workload_suffix = "-fp16.json"

    workload_path = f"{CUR_DIR}/out/workloads/{model_id}-{dataset}-{bs}{workload_suffix}"
    trace = trace or MODEL_ID_TO_TRACE_FILE[model_id][dataset]
    if not os.path.exists(trace):
        print(f"trace file `{trace}` not found: pass --trace PATH or --synthetic {{c1..c5}}", file=sys.stderr)
        return 2
    layers = list(range(MODEL_ID_TO_LAYERS[model_id])) if layer == -1 else [layer]

    from mxmoe_amd import harness

    # the kernel library depends on the format set only: generate and build it once, not per layer
    print(f"qcfg_list: {sorted(qcfg_list)}")
    gpu_info = get_gpu_info()
    tile_configs = None
    if args.tile_config is not None:
        with open(args.tile_config) as f:
            tile_configs = load_tile_configs(json.load(f), qcfg_list)
    generator = TemplateGenerator(gpu_info["cc"], qcfg_list, KernelType.Fused, tile_configs)
    if args.max_kernels:
        combos = generator.get_tile_configs()[: args.max_kernels]
        generator.get_tile_configs = lambda: combos
    generator.generate_source_code()
    lib_path = generator.build()

    from mxmoe_amd import _lib

    if args.no_bench:
        for lyr in layers:
            generate_workload_from_gate_trace(trace, bs, lyr, workload_path, args.qconfig, args.qstr if args.qconfig is None else None, exact_counts=exact)
        print(f"workload: {workload_path}\nlibrary: {lib_path}")
        return 0
    lib = _lib.load(lib_path)
    os.makedirs(f"{CUR_DIR}/out/bench", exist_ok=True)
    bench_save = f"{CUR_DIR}/out/bench/{model_id}-{dataset}-{bs}{workload_suffix.replace('.json', '')}"
    for lyr in layers:
        generate_workload_from_gate_trace(trace, bs, lyr, workload_path, args.qconfig, args.qstr if args.qconfig is None else None, exact_counts=exact)
        harness.bench_input_file(workload_path, bench_save, lib=lib, mode=args.mode)
    return 0


if __name__ == "__main__":
    sys.exit(main())
