"""Bench / check harness over workload JSON files: the Python port of the reference's C++ `test` program
(mxmoe/kernels/src/test.cu: parse_json_input :652-674, QInput::from_fp16 :218-413, bench_one_case :693-868,
bench_input_file :870-946; timing protocol mxmoe/kernels/src/test_utils.h:97-191; check tolerance :70-95).

Per (layer, "gate_up" | "down") problem list: fp16 operands ~ U(-1, 1) (seed 42), operands quantised + packed per problem,
every registered fused kernel that covers the formats is timed (<= 30 warm-up, <= 50 timed launches, HIP events, median)
and reported as `kernel_name, avg_time (ms), TFLOPS, speedup` against the best fp16 grouped GEMM of the same shapes (the
reference's CUTLASS baseline; here the fp16 MFMA kernel), written to `<output>-layer-<i>-<gate_up|down>.csv`.
Sequential and multi-stream launches (one launch per contiguous run of equal-format problems, on one stream or dealt to
side streams — the reference's ablation launchers, kernel_sketch.py:148-406, here policies of the C++ host launcher) are
timed next to the fused launch.
"""
from __future__ import annotations

import json
import time

import torch

from . import _lib, pack
from .group_gemm import GroupGemmLaunch
from .quant import quant_minmax
from .weights import quantize_and_pack


def parse_json_input(path: str) -> dict:
    """test.cu:652-674: {case name: {"gate_up": [...], "down": [...]}} with entries {"shape": [M, N, K], "w_bits", "a_bits", "gsize",
    "sym"}; every top-level key except "num_tokens" is a case (the workload generator writes "layer-<i>")."""
    with open(path) as f:
        data = json.load(f)
    return {k: v for k, v in data.items() if k != "num_tokens"}


def parse_legacy_input(path: str) -> dict:
    """test.cu:611-650: a text file with one problem per line, `a_bits-w_bits-gsize-{sym|asym} MxNxK` (any single character between the
    numbers), all of them one problem list `{"test_case": {"gate_up": [...]}}`.  Weight bits 16 / 8 / 4 / 2 and activation bits
    16 / 8 / 4, as there."""
    import re

    shapes = []
    with open(path) as f:
        for line in f:
            if not line.strip():
                continue
            m = re.match(r"\s*(\d+)\D(\d+)\D(-?\d+)\D(sym|asym)\s+(\d+)\D(\d+)\D(\d+)\s*$", line)
            if not m:
                raise ValueError(f"cannot parse `{line.rstrip()}`: expected `a_bits-w_bits-gsize-sym MxNxK`")
            a_bits, w_bits, gsize = int(m.group(1)), int(m.group(2)), int(m.group(3))
            if w_bits not in (16, 8, 4, 2):
                raise ValueError(f"Ava w bits: [16, 8, 4, 2]. Got {w_bits}")
            if a_bits not in (16, 8, 4):
                raise ValueError(f"Ava a bits: [16, 8, 4]. Got {a_bits}")
            shapes.append({"shape": [int(m.group(5)), int(m.group(6)), int(m.group(7))], "w_bits": w_bits, "a_bits": a_bits, "gsize": gsize, "sym": m.group(4) == "sym"})
    return {"test_case": {"gate_up": shapes}}


def parse_input_file(path: str) -> dict:
    """test.cu:676-691: a `.json` workload file or a legacy text file."""
    import os

    if not os.path.exists(path):
        raise FileNotFoundError(f"input file: `{path}` not found")
    return parse_json_input(path) if str(path).endswith(".json") else parse_legacy_input(path)


def bench_func(fn, warmup: int = 20, iters: int = 50, max_warm_s: float = 10.0) -> dict:
    """test_utils.h:97-191: warm-up (bounded by count and time), then `iters` launches timed one by one with device events;
    returns min / max / trimmed mean / median in milliseconds (the reference reports the median)."""
    t0 = time.time()
    for _ in range(warmup):
        fn()
        if time.time() - t0 > max_warm_s:
            break
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in ev)
    trim = ts[len(ts) // 10: len(ts) - len(ts) // 10] or ts
    return {"min": ts[0], "max": ts[-1], "mean": sum(trim) / len(trim), "median": ts[len(ts) // 2]}


def make_problem(entry: dict, gen: torch.Generator, device="cuda", keep_ref: bool = False, bf6: bool = False, fp8: bool = False, bf16: bool = False) -> dict:
    """Random fp16 operands for one workload entry, quantised and packed for its format (QInput::from_fp16).  `bf6`: w4a4 operands as
    bf6 fragments, the layout of the kernels whose w4a4 tiles run on the 6-bit float matrix path (`kernel_takes_bf6`).  `bf16`: the
    16-bit float problems hold bfloat16 numbers (kernels whose dense tiles run the bf16 matrix instruction); their tensors keep the
    fp16 dtype as a container of the bits (`.view(torch.bfloat16)` reads them)."""
    m, n, k = entry["shape"]
    qp = (entry["a_bits"], entry["w_bits"], entry["gsize"], bool(entry["sym"]))
    if gen is None:  # values drawn on the device (timing-only problems)
        a = torch.rand(m, k, dtype=torch.float16, device=device) * 2 - 1
        b = torch.rand(n, k, dtype=torch.float16, device=device) * 2 - 1
    else:
        a = (torch.rand(m, k, generator=gen, dtype=torch.float32) * 2 - 1).to(torch.float16).to(device)
        b = (torch.rand(n, k, generator=gen, dtype=torch.float32) * 2 - 1).to(torch.float16).to(device)
    fp8 = fp8 and qp[:3] == (8, 8, -1)
    if bf16 and qp[0] >= 16 and qp[1] >= 16:
        a, b = a.to(torch.bfloat16), b.to(torch.bfloat16)
        prob = {"size": (m, n, k), "q": qp, "A": a.view(torch.float16), "sa": None, "B": b.view(torch.float16), "sb": None,
                "C": torch.zeros(m, n, dtype=torch.float16, device=device), "bf16": True}
        if keep_ref:
            prob["a16"], prob["b16"] = a, b
        return prob
    pw = quantize_and_pack(b, qp, bf6=bf6, fp8=fp8)
    prob = {"size": (m, n, k), "q": qp, "B": pw.data, "sb": pw.scale, "C": torch.zeros(m, n, dtype=torch.float16, device=device)}
    if qp[0] < 16:
        ag = qp[2] if qp[2] > 0 else -1                      # group-quantised activations (w4a4_g128_sym): scales [M, K / 128]
        if fp8:
            from .quant import quant_e4m3

            qa, sa = quant_e4m3(a) if m else (a.view(torch.uint8)[:, :k], a[:, :1])
            qi = qa.reshape(m, k).view(torch.int8)
        else:
            qa, sa, _ = quant_minmax(a, qp[0], ag, True) if m else (a, a[:, :1], None)
            qi = qa.reshape(m, k).to(torch.int8)
        prob["A"] = qi.contiguous() if qp[0] == 8 else (pack.pack_bf6_fragments(qi) if bf6 and qp[2] == -1 and qp[1] == 4 else pack.pack_int4_k(qi))
        prob["sa"] = sa.reshape(-1).contiguous()
    else:
        prob["A"], prob["sa"] = a, None
    if keep_ref:
        prob["a16"], prob["b16"] = a, b
    return prob


def kernel_takes_bf6(lib, kid: int) -> bool:
    """Whether kernel `kid` has w4a4 tiles on the 6-bit float matrix path: its w4a4 operands are bf6 fragments."""
    from .ops import kernel_variants

    return kernel_variants(lib, kid).get(2) == 1


def kernel_takes_fp8(lib, kid: int) -> bool:
    """Whether kernel `kid` runs its w8a8 problems on the fp8 instruction: their operands are e4m3 codes, not int8 ones."""
    from .ops import kernel_variants

    return kernel_variants(lib, kid).get(1) == 2


def kernel_takes_bf16(lib, kid: int) -> bool:
    """Whether kernel `kid` computes its 16-bit float problems in bfloat16."""
    from .ops import kernel_variants

    return kernel_variants(lib, kid).get(0) == 3


def _launch_of(probs, lib, kernel_id=-1) -> GroupGemmLaunch:
    return GroupGemmLaunch([p["A"] for p in probs], [p["B"] for p in probs], [p["sa"] for p in probs], [p["sb"] for p in probs],
                           [p["C"] for p in probs], [p["size"] for p in probs], [p["q"] for p in probs], kernel_id=kernel_id, lib=lib)


def _runs_of_equal_format(probs):
    runs, cur = [], []
    for p in probs:
        if cur and p["q"] != cur[-1]["q"]:
            runs.append(cur)
            cur = []
        cur.append(p)
    if cur:
        runs.append(cur)
    return runs


POLICY_KERNEL = {"seq": b"groupgemm_seq_launch_all", "ms": b"groupgemm_ms_launch_all"}


def launch_policy(probs, policy: str, lib=None):
    """A callable that runs the problem list once under `policy`: "fused" (one launch, the library's first kernel that covers the
    formats), "seq" or "ms" (the default library's sequential / multi-stream launchers, the reference's ablation baselines
    kernel_sketch.py:148-406: one launch per run of consecutive equal-format problems, on the current stream or on the
    library's side streams)."""
    if policy == "fused":
        g = _launch_of(probs, lib or _lib.load())
    else:
        lib = _lib.load()
        kid = lib.mxmoe_find_kernel(POLICY_KERNEL[policy])
        if kid < 0 or lib.mxmoe_kernel_policy(kid) != {"seq": 1, "ms": 2}[policy]:
            raise RuntimeError(f"the library has no {policy} launcher")
        g = _launch_of(probs, lib, kid)
    g.plan()
    return g.run


def tflops(probs, ms: float) -> float:
    return sum(2 * m * n * k for (m, n, k) in (p["size"] for p in probs)) / (ms * 1e-3) / 1e12


def bench_one_case(entries, lib=None, mode: str = "bench", filters=(), out_file: str | None = None, verbose: bool = False) -> dict:
    """Time (or check) every registered kernel on one problem list; returns {impl: (avg_time_ms, TFLOPS, kernel_name)}."""
    lib = lib or _lib.load()
    default_lib = _lib.load()
    gen = torch.Generator(device="cpu")
    gen.manual_seed(42)
    probs = [make_problem(e, gen, keep_ref=(mode == "check")) for e in entries]
    probs = [p for p in probs if p["size"][0] > 0]
    variants = {}    # the same problems with operand variants (w4a4 as bf6 fragments, w8a8 as fp8 codes), made when a kernel asks for them

    # fp16 baseline on the same shapes (role of the CUTLASS grouped GEMM, test.cu:774-781)
    gen2 = torch.Generator(device="cpu")
    gen2.manual_seed(42)
    base_probs = [make_problem({**e, "a_bits": 16, "w_bits": 16, "gsize": -1, "sym": True}, gen2) for e in entries if e["shape"][0] > 0]
    base = _launch_of(base_probs, default_lib)
    base_ms = bench_func(base.run)["median"]
    results = {"fp16-baseline": (base_ms, tflops(base_probs, base_ms), default_lib.mxmoe_kernel_name(base.plan()[0]).decode())}

    rows = []
    for kid in range(lib.mxmoe_num_kernels()):
        name = lib.mxmoe_kernel_name(kid).decode()
        if filters and not any(f in name for f in filters):
            continue
        mine = probs
        want = (kernel_takes_bf6(lib, kid) and any(p["q"][:3] == (4, 4, -1) for p in probs), kernel_takes_fp8(lib, kid) and any(p["q"][:3] == (8, 8, -1) for p in probs),
                kernel_takes_bf16(lib, kid) and any(p["q"][0] >= 16 and p["q"][1] >= 16 for p in probs))
        if any(want):
            if want not in variants:
                gen.manual_seed(42)
                variants[want] = [make_problem(e, gen, keep_ref=(mode == "check"), bf6=want[0], fp8=want[1], bf16=want[2]) for e in entries if e["shape"][0] > 0]
            mine = variants[want]
        g = _launch_of(mine, lib, kid)
        try:
            g.plan()
        except RuntimeError:
            continue  # this kernel has no tile for one of the formats (or does not take one of the shapes)
        if mode == "check":
            g.run()
            torch.cuda.synchronize()
            for p in mine:
                ref = (p["a16"].float() @ p["b16"].float().T)
                got = p["C"].view(torch.bfloat16) if p.get("bf16") else p["C"]
                err = (got.float() - ref).abs().max().item() if p["size"][0] else 0.0
                tol = 1.0 if p["q"][1] >= 16 else float("inf")  # test_utils.h:71 — meaningful for fp16 only, as in the reference
                print(f"{name}: problem {p['size']} {p['q']} max abs err vs fp16 reference {err:.4f}{' FAIL' if err > tol else ''}")
            continue
        ms = bench_func(g.run)["median"]
        rows.append((ms, tflops(probs, ms), name))
        if verbose:
            print(f"{name}\navg_time: {ms:<8.4f}, TFLOPS: {tflops(probs, ms):<9.4f}")
        time.sleep(0.05)
    if mode == "check":
        return results

    if rows:
        results["mxmoe-hz"] = min(rows)
    # ablation launch policies (the library's sequential and multi-stream launchers over the same tiles)
    for impl, policy in (("mxmoe-seq", "seq"), ("mxmoe-ms", "ms")):
        try:
            run = launch_policy(probs, policy)
        except RuntimeError:
            continue  # a format outside the every-format kernel
        ms = bench_func(run)["median"]
        results[impl] = (ms, tflops(probs, ms), f"{policy}_launch x{len(_runs_of_equal_format(probs))}")

    base_tf = results["fp16-baseline"][1]
    for impl, (ms, tf, name) in results.items():
        print(f"{impl}: {name}\navg_time: {ms:<8.4f}, TFLOPS: {tf:<9.4f}, speedup: {tf / base_tf:<.3f}")
    if out_file:
        with open(out_file, "w") as f:
            f.write("kernel_name,avg_time,TFLOPS,speedup\n")
            for ms, tf, name in rows:
                f.write(f"\"{name}\",{ms:.4f},{tf:.4f},{tf / base_tf:.3f}\n")
    return results


def bench_input_file(input_path: str, output_prefix: str | None = None, lib=None, mode: str = "bench", filters=(), verbose: bool = False) -> dict:
    """test.cu:870-946: every case of the input file (the layers of a workload file, gate_up then down; the one list of a legacy
    file), one CSV per problem list named `<output>-<case>-<gate_up|down>.csv` (test.cu:942)."""
    out = {}
    for case, lists in parse_input_file(input_path).items():
        for which in ("gate_up", "down"):
            if which not in lists:
                continue
            csv = f"{output_prefix}-{case}-{which}.csv" if output_prefix else None
            print(f"== {case} {which}: {len(lists[which])} problems")
            out[(case, which)] = bench_one_case(lists[which], lib=lib, mode=mode, filters=filters, out_file=csv, verbose=verbose)
    return out
