"""Expert-frequency trace + qconfig -> per-layer GroupGEMM problem list (the workload JSON).

Same behaviour and JSON shape as the reference's `generate_workload_from_gate_trace` (mxmoe/kernels/gen_workload.py:31-103),
including its quirks: `M_e = int(p_e * T * topk)` (floors), the shared expert is one problem `[T, 2N*n_shared, K]` /
`[T, K, N*n_shared]` stored as expert index E, and its `down` problem takes the "gate" block's qcfg (:93-94).
"""
from __future__ import annotations

import argparse
import json
import os

from ..project_config import CUR_DIR

MODEL_ID_TO_LAYERS = {"qwen2_moe": 24, "qwen2_moe_57b": 28, "ds2": 27, "mixtral": 32}

MODEL_ID_TO_TRACE_FILE = {
    k: {d: f"{CUR_DIR}/calib/gate/{k}/{d}/4096/moe-gate.json" for d in ["wiki2", "humaneval-x", "synthetic"]}
    for k in ["qwen2_moe", "qwen2_moe_57b", "ds2", "mixtral"]
}


def freq_to_prob(freq):
    total = sum(freq)
    return [f / total for f in freq]


def parse_qstr(qstr: str) -> dict:
    return {
        "w_bits": int(qstr.split("w")[1].split("a")[0]),
        "a_bits": int(qstr.split("a")[1].split("_g")[0]),
        "gsize": int(qstr.split("_g")[1].split("_")[0]),
        "sym": "asym" not in qstr,
    }


def generate_workload_from_gate_trace(trace_file: str, num_total_tokens: int, layer_id: int, save_path: str | None, qcfg_file=None, qstr=None, exact_counts: bool = False) -> dict:
    assert trace_file.endswith(".json") and os.path.exists(trace_file), trace_file
    assert qcfg_file is None or qstr is None
    qconfig = None
    if qcfg_file is not None:
        assert qcfg_file.endswith(".json") and os.path.exists(qcfg_file)
        with open(qcfg_file) as f:
            qconfig = json.load(f)
        qconfig.pop("LT", None)
        qcfg = None
    elif qstr is not None and qstr != "fp16":
        qcfg = parse_qstr(qstr)
    else:
        qcfg = {"w_bits": 16, "a_bits": 16, "gsize": -1, "sym": True}

    with open(trace_file) as f:
        trace = json.load(f)
    topk = trace["topk"]
    n, k = trace["NK"]
    num_shared = trace["num_shared_experts"]
    result = {"num_tokens": num_total_tokens}
    for key, value in trace.items():
        if not key.startswith("layer-"):
            continue
        layer_idx = key.split("-")[1]
        if layer_id != -1 and layer_idx != str(layer_id):
            continue

        def block_qcfg(exp_idx: str, linear: str) -> dict:
            if qconfig is None:
                return qcfg
            c = qconfig[layer_idx]["experts"][exp_idx][linear]
            return {"w_bits": c["w_bits"], "a_bits": c["a_bits"], "gsize": c["w_gsize"], "sym": c["w_sym"]}

        freq = value["access_freq"]
        num_experts = len(freq)
        prob = freq_to_prob(freq)
        exact = exact_counts and sum(freq) == num_total_tokens * topk
        shapes = {"gate_up": [], "down": []}
        for e, p in enumerate(prob):
            m = int(freq[e]) if exact else int(p * num_total_tokens * topk)
            shapes["gate_up"].append({"shape": [m, n * 2, k], **block_qcfg(str(e), "gate")})
            shapes["down"].append({"shape": [m, k, n], **block_qcfg(str(e), "down")})
        if num_shared != 0:
            shapes["gate_up"].append({"shape": [int(num_total_tokens), n * 2 * num_shared, k], **block_qcfg(str(num_experts), "gate")})
            shapes["down"].append({"shape": [int(num_total_tokens), k, n * num_shared], **block_qcfg(str(num_experts), "gate")})
        result[f"layer-{layer_idx}"] = shapes

    if save_path is not None:
        os.makedirs(os.path.dirname(save_path) or ".", exist_ok=True)
        with open(save_path, "w") as f:
            f.write(json.dumps(result, indent=2))
        print(f"Save generated workloads to `{save_path}`")
    return result


def main(argv=None) -> int:
    p = argparse.ArgumentParser(description="Generate workloads for groupgemm kernel.")
    p.add_argument("--model", type=str, default="qwen2_moe")
    p.add_argument("--dataset", type=str, default="wiki2")
    p.add_argument("--length", type=int, default=128)
    p.add_argument("--scale", type=float, nargs="+", default=[1.0])
    p.add_argument("--layer", type=int, default=-1)
    p.add_argument("--qconfig", type=str)
    p.add_argument("--qstr", type=str)
    p.add_argument("--save", type=str)
    p.add_argument("--trace", type=str, default=None, help="trace file (default: the reference's calib/gate/... path)")
    a = p.parse_args(argv)
    trace = a.trace or MODEL_ID_TO_TRACE_FILE[a.model][a.dataset]
    print(f"Generate workloads from `{trace}` with scale: {a.scale}")
    for s in a.scale:
        generate_workload_from_gate_trace(trace, int(a.length * s), a.layer, a.save, a.qconfig, a.qstr)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
