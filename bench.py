#!/usr/bin/env python3
"""GroupGEMM benchmark of the mixed-precision MoE layer on one MI355X.

One "step" = the two fused GroupGEMM launches of one MoE layer (gate_up, then down) over one batch of synthetic,
HBM-resident, already permuted + quantised inputs — the region the reference times with cudaEvents around its launcher
(mxmoe/kernels/src/test.cu:101-158, mxmoe/kernels/src/test_utils.h:97-191), metric TOPS = sum(2*M*N*K) / time.

Prints ONE JSON line.  `roofline` prices the dominant kernel (the gate_up launch) against the MI355X peak with its launch
duration measured by HIP events on the launch stream inside the timed region; `cpu_baseline` times the CPU restatement of
the reference's fake-quant path on a bounded sample of the same workload on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

PEAK = {"int8": 5000.0, "fp16": 2500.0, "fp6": 10100.0, "hbm": 8000.0}  # MI355X: TOP/s dense int8 MFMA, TFLOP/s dense fp16 / fp6 MFMA, GB/s HBM3E

# HBM bytes per launch of the dominant (gate_up) kernel, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs scaled by the
# same counters on a plain 256 MiB copy (summaries: profiles/fused_group_gemm_<workload>.txt, profiles/counter_calibration_copy_256MiB.txt)
TRAFFIC = {"c1": 729899884, "c2": 556661594, "c3": 684746679, "c4": 201769125, "c5": 5813884599}


def build_layer(name: str, tokens: int | None, bf6=False):
    import torch

    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.get_config(name, tokens)
    hidden = synth.make_hidden(cfg)
    ids, _ = synth.make_routing(cfg)
    layer = MxMoELayer(cfg, bf6=bf6)
    layer.prepare(hidden, ids)
    layer.gate_up()
    layer.act()
    layer.down()
    torch.cuda.synchronize()
    return cfg, layer


def time_layer(layer, steps: int, warmup: int, settle_s: float = 0.15):
    """K steps of (gate_up launch, down launch); returns (ms_per_step, avg gate_up ms, avg down ms).

    The timed region holds nothing but the 2K launches (events between launches open gaps of several microseconds, which are not
    part of the work); the per-launch durations are taken in a second, instrumented pass of the same K steps."""
    import torch

    st = layer.state
    g1, g2 = st["gg1"], st["gg2"]
    # After an idle period the GPU needs tens of milliseconds of continuous work to reach its sustained clock; bring it there
    # before the warm-up steps, whatever their number, so that a short --warmup does not time the ramp.
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_s:
        for _ in range(20):
            g1.run()
            g2.run()
        torch.cuda.synchronize()
    for _ in range(warmup):
        g1.run()
        g2.run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        g1.run()
        g2.run()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for a, b, c in ev:
        a.record()
        g1.run()
        b.record()
        g2.run()
        c.record()
    torch.cuda.synchronize()
    up = sum(a.elapsed_time(b) for a, b, _ in ev) / steps
    dn = sum(b.elapsed_time(c) for _, b, c in ev) / steps
    return wall / steps, up, dn


def launch_duration(plan, n: int = 20, warm: int = 100) -> float:
    """Average duration (ms) of one launch: n back-to-back launches between two HIP events on the launch stream (no event
    between launches, so dispatch gaps of a few microseconds do not count as kernel time)."""
    import torch

    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(warm):  # the GPU needs tens of milliseconds of continuous work to settle at its sustained clock
        plan.run()
    a.record()
    for _ in range(n):
        plan.run()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n


def _default_tokens(name: str) -> int:
    from mxmoe_amd import synth

    return synth.CONFIGS[name].tokens if name in synth.CONFIGS else -1


def roofline_entry(cfg, layer, name: str) -> dict:
    """Roofline entry of one launch ("gate_up" or "down").  Compute-bound layers (w-a formats at thousands of tokens): ops of the
    launch against the int8 (or fp16) MFMA peak.  Skinny weight-only layers: algorithmic bytes against HBM."""
    st = layer.state
    by = layer.algorithmic_bytes()
    plan = st["gg1"] if name == "gate_up" else st["gg2"]
    ms = launch_duration(plan)
    traffic = TRAFFIC.get(cfg.name) if name == "gate_up" and cfg.tokens == _default_tokens(cfg.name) else None
    # `traffic` is not measured by this run: it is the figure of the rocprofv3 --pmc summary named here (same command, same seeds)
    src = {"traffic_source": f"profiles/fused_group_gemm_{cfg.name}.txt"} if traffic is not None else {}
    fmts = {q[:2] for q in plan.qparams}
    compute_bound = cfg.tokens * cfg.topk / cfg.num_experts >= 128
    if compute_bound:
        peak = PEAK["fp16"] if all(a >= 16 for a, _ in fmts) else PEAK["int8"]
        ach = plan.ops / (ms * 1e-3) / 1e12
        return {"kernel": f"fused_group_gemm[{name}]", "bound": "mfma", "achieved": round(ach, 2), "peak": peak, "unit": "TFLOP/s",
                "frac": round(ach / peak, 4), "traffic": traffic, **src, "launch_us": round(ms * 1e3, 2), "algorithmic_bytes": by[name]["total"]}
    ach = by[name]["total"] / (ms * 1e-3) / 1e9
    return {"kernel": f"fused_group_gemm[{name}]", "bound": "hbm", "achieved": round(ach, 1), "peak": PEAK["hbm"], "unit": "GB/s",
            "frac": round(ach / PEAK["hbm"], 4), "traffic": traffic, **src, "launch_us": round(ms * 1e3, 2), "algorithmic_bytes": by[name]["total"]}


def roofline_of(cfg, layer, up_ms: float, dn_ms: float):
    """(entry of the dominant launch, entry of the other launch)."""
    names = ("gate_up", "down") if up_ms >= dn_ms else ("down", "gate_up")
    return tuple(roofline_entry(cfg, layer, n) for n in names)


def roofline_step(cfg, layer, ms: float) -> dict:
    """The whole step (both launches back to back on one stream, `ms` per step by the bench's own clock) against the same peak as
    its launches: ops of both over the step time, or algorithmic bytes of both for the few-token weight-only layers."""
    st = layer.state
    by = layer.algorithmic_bytes()
    fmts = {q[:2] for plan in (st["gg1"], st["gg2"]) for q in plan.qparams}
    if cfg.tokens * cfg.topk / cfg.num_experts >= 128:
        peak = PEAK["fp16"] if all(a >= 16 for a, _ in fmts) else PEAK["int8"]
        ach = layer.gemm_ops() / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": round(ach, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(ach / peak, 4), "step_us": round(ms * 1e3, 2)}
    total = by["gate_up"]["total"] + by["down"]["total"]
    ach = total / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": round(ach, 1), "peak": PEAK["hbm"], "unit": "GB/s", "frac": round(ach / PEAK["hbm"], 4), "step_us": round(ms * 1e3, 2),
            "algorithmic_bytes": total}


def cpu_baseline(cfg, budget_s: float = 20.0):
    """The fake-quant path (per expert: fake_quant(x) @ fake_quant(W13)^T -> SiLU*up -> fake_quant(.) @ fake_quant(W2)^T,
    fp16 storage, fp32 matmul) from the CPU oracle, on as many experts of this workload as fit the time budget."""
    import numpy as np

    from mxmoe_amd import synth
    from oracle import mxmoe_oracle as O

    hidden = synth.make_hidden(cfg).numpy()
    ids, _ = synth.make_routing(cfg)
    _, perm, _, recv = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    formats = synth.draw_formats(cfg)
    starts = np.concatenate([[0], np.cumsum(recv)])
    ops = 0
    spent = 0.0
    used = []
    f32 = np.float32
    for e in np.argsort(-recv):  # busiest experts first
        m = int(recv[e])
        if m == 0 or spent > budget_s:
            break
        w13, w2 = (w.numpy() for w in synth.expert_weights(cfg, int(e)))
        (a1, wb1, g1, s1), (a2, wb2, g2, s2) = formats[e]
        w13q = O.fake_quant(w13, wb1, g1, s1).astype(f32)  # offline in the reference (quant.py:913): not timed
        w2q = O.fake_quant(w2, wb2, g2, s2).astype(f32)
        x = hidden[perm[starts[e]:starts[e + 1]]]
        t0 = time.perf_counter()
        xq = O.fake_quant(O.online_hadamard(x) if (cfg.rotate and a1 < 16) else x, a1, -1, True) if a1 < 16 else x
        mid = (xq.astype(f32) @ w13q.T).astype(np.float16)
        y = O.silu_mul(mid)
        yq = O.fake_quant(O.online_hadamard(y) if (cfg.rotate and a2 < 16) else y, a2, -1, True) if a2 < 16 else y
        out = (yq.astype(f32) @ w2q.T).astype(np.float16)
        spent += time.perf_counter() - t0
        assert out.shape == (m, cfg.hidden)
        ops += 2 * m * (2 * cfg.inter * cfg.hidden + cfg.hidden * cfg.inter)
        used.append(int(e))
    cores = os.cpu_count() or 1
    try:  # the threads the BLAS behind numpy actually runs (the box caps them below the core count)
        from threadpoolctl import threadpool_info

        blas = [int(p["num_threads"]) for p in threadpool_info() if p.get("user_api") == "blas"]
        cores = max(blas) if blas else cores
    except ImportError:
        pass
    return {"value": round(ops / spent / 1e12, 5), "unit": "TOPS", "cores": cores, "kind": "port",
            "sample": f"{len(used)} busiest experts of {cfg.name} ({sum(int(recv[e]) for e in used)} of {cfg.rows} routed rows), "
                      f"activation fake-quant + fp32 matmuls + SiLU timed, {spent:.1f} s"}


def time_whole_layer(cfg, layer, reps: int = 7) -> dict:
    """Wall time of the whole layer forward as a caller of the ops sees it (permute + rotate + quantise, gate_up launch, SiLU*up +
    rotate + quantise, down launch, un-permute + combine), including the host work of the ops (offset tables, allocations); median of
    `reps` repetitions, step by step with a synchronisation after each (`*_ms`, `layer_ms`) and as the layer's one-call form (`one_call_ms`).
    Reported next to the GroupGEMM figure, never as `value`."""
    import torch

    from mxmoe_amd import synth

    hidden = synth.make_hidden(cfg).cuda()
    ids, w = synth.make_routing(cfg)
    ids, w = ids.cuda(), w.cuda()
    names = ("prologue", "gate_up", "act", "down", "combine")
    samples = {k: [] for k in names}
    for rep in range(reps + 2):
        torch.cuda.synchronize()
        marks = [time.perf_counter()]
        for fn in (lambda: layer.prepare(hidden, ids), layer.gate_up, layer.act, layer.down, lambda: layer.combine(w)):
            fn()
            torch.cuda.synchronize()
            marks.append(time.perf_counter())
        if rep >= 2:  # the first repetitions settle the allocator
            for k, a, b in zip(names, marks, marks[1:]):
                samples[k].append((b - a) * 1e3)
    parts = {k: sorted(v)[len(v) // 2] for k, v in samples.items()}
    out = {f"{k}_ms": round(v, 4) for k, v in parts.items()}
    out["layer_ms"] = round(sum(parts.values()), 4)
    # the same forward as one call: tables planned on the device, no synchronisation, persistent buffers
    out_buf = torch.empty((cfg.tokens, cfg.hidden), dtype=torch.float16, device="cuda")

    def wall(fn):
        ts = []
        for rep in range(reps + 2):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            ts.append((time.perf_counter() - t0) * 1e3)
        ts = sorted(ts[2:])
        return round(ts[len(ts) // 2], 4)

    out["one_call_ms"] = wall(lambda: layer(hidden, ids, w, out=out_buf))
    out["one_call_host_tables_ms"] = wall(lambda: layer.call_with_host_tables(hidden, ids, w))   # tables built on the host after reading the counts back
    # ... and replayed from a HIP graph
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(hidden, ids, w, out=out_buf)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer(hidden, ids, w, out=out_buf)
    out["graph_replay_ms"] = wall(graph.replay)
    return out


def run_workload(name: str, steps: int, warmup: int, tokens=None, whole: bool = True, bf6=False):
    cfg, layer = build_layer(name, tokens, bf6)
    ms, up, dn = time_layer(layer, steps, warmup)
    ops = layer.gemm_ops()
    st = layer.state
    roof = roofline_of(cfg, layer, up, dn)
    return cfg, layer, {
        "workload": name, "tops": round(ops / (ms * 1e-3) / 1e12, 2), "ms_per_step": round(ms, 4),
        "gate_up_us": round(up * 1e3, 2), "down_us": round(dn * 1e3, 2),
        "gate_up_tops": round(st["gg1"].ops / (up * 1e-3) / 1e12, 2), "down_tops": round(st["gg2"].ops / (dn * 1e-3) / 1e12, 2),
        "ops": ops, "whole_layer": time_whole_layer(cfg, layer) if whole else None, "roofline": roof[0], "roofline_other_launch": roof[1],
        "roofline_step": roofline_step(cfg, layer, ms),
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c3", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--also", default="c2,c4", help="comma-separated extra workloads reported under 'also' (empty to skip)")
    ap.add_argument("--tokens", type=int, default=None)
    ap.add_argument("--w4a4-path", default="int8", choices=["bf6", "int8", "bf6-down"],
                    help="matrix instruction of the w4a4 blocks: int8 = v_mfma_i32_32x32x32_i8 on codes widened in registers, bf6 = "
                         "v_mfma_scale_f32_32x32x64_f8f6f4 on int4 values held as 6-bit floats (exact), bf6-down = bf6 for the down blocks only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-whole-layer", action="store_true", help="skip the wall-clock timing of the whole forward (profiling runs: the trace then ends with the launches the roofline entry is measured on)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="instead of the benchmark, run a plain device copy of BYTES bytes 5 times (reference point for the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the layer would shard by expert, one all-to-all of rows either side of the launches). Use --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the HIP kernels)", file=sys.stderr)
        return 2
    if args.copy_calibration:
        src = torch.empty(args.copy_calibration, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": args.copy_calibration, "copies": 5}))
        return 0
    from mxmoe_amd import synth

    bf6 = {"int8": False, "bf6": True, "bf6-down": (False, True)}[args.w4a4_path]
    cfg, layer, main_res = run_workload(args.workload, args.steps, args.warmup, args.tokens, not args.no_whole_layer, bf6)
    also = {}
    del layer
    torch.cuda.empty_cache()
    for extra in [w for w in args.also.split(",") if w and w != args.workload]:
        _, lay, res = run_workload(extra, max(10, args.steps // 2), max(5, args.warmup // 2), whole=not args.no_whole_layer, bf6=bf6)
        also[extra] = res
        del lay
        torch.cuda.empty_cache()

    # the same workload with its w4a4 blocks on the other matrix instruction (same codes, same results bit for bit), for comparison
    alt = None
    if any(tuple(q) == synth.W4A4 for f in synth.draw_formats(cfg) for q in f) and args.tokens is None:
        other = "int8" if args.w4a4_path != "int8" else "bf6"
        _, lay, res = run_workload(args.workload, max(10, args.steps // 2), max(5, args.warmup // 2), whole=False, bf6=other == "bf6")
        alt = {"w4a4_path": other, **{k: res[k] for k in ("tops", "ms_per_step", "gate_up_us", "down_us")},
               "gate_up_launch_us": res["roofline"]["launch_us"], "down_launch_us": res["roofline_other_launch"]["launch_us"]}
        del lay
        torch.cuda.empty_cache()
    fm = sorted({synth.qcfg_str(q) for f in synth.draw_formats(cfg) for q in f})
    out = {
        "metric": "GroupGEMM TOPS, Qwen1.5-MoE layer bs=8192" if args.workload in ("c2", "c3") else f"GroupGEMM TOPS, {cfg.description}",
        "value": main_res["tops"],
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if any(q != "fp16" and "a16" not in q for q in fm) else "f16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {cfg.description}", "experts": cfg.num_experts, "topk": cfg.topk, "hidden": cfg.hidden,
                   "intermediate": cfg.inter, "tokens": cfg.tokens, "formats": fm, "step": "gate_up GroupGEMM launch + down GroupGEMM launch"},
        "roofline": main_res["roofline"],
        "detail": {**{k: main_res[k] for k in ("gate_up_us", "down_us", "gate_up_tops", "down_tops", "ops", "whole_layer", "roofline_other_launch", "roofline_step")},
                   "w4a4_path": args.w4a4_path, "other_w4a4_path": alt},
        "also": also,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
