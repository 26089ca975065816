"""Offline weight pipeline and on-disk format of one MoE layer.

fp16 expert weights (a `state_dict` in the model family's naming) + the qconfig of the layer  ->  weights rotated for the online
Hadamard transform, RTN-quantised and packed in the kernels' layouts  ->  one safetensors file that `load_layer` maps straight
into the tensors the GroupGEMM launch reads.  Counterpart of the reference's offline steps: weight lookup by family
(mxmoe/quant/moe_utils.py:36-63, 188-207), rotation of the MLP input weights `W <- W Q` in fp64 (mxmoe/quant/rotation.py:353-364),
RTN quantisation (mxmoe/quant/quant.py:40-109) and packing (mxmoe/kernels/src/include/quantize.cuh:383-475; own gfx950 layouts here).

File layout (safetensors): tensors `e{idx}.w13.data`, `e{idx}.w13.scale`, `e{idx}.w2.data`, `e{idx}.w2.scale` (the shared experts,
fused into one expert, are index `num_experts`); metadata `mxmoe_layer` = JSON {format, model, layer, num_experts, num_shared, hidden,
inter, rotate, experts: [{gate_up: [a_bits, w_bits, gsize, sym], down: [...], n13, k13, n2, k2}]}.
"""
from __future__ import annotations

import json

import numpy as np
import torch

from .hadamard import get_hadK
from .weights import PackedWeight, pack_codes, quantize_and_pack

FORMAT_VERSION = 1
MOE_MLP_NAME_MAP = {"ds2": "mlp", "qwen2_moe": "mlp", "qwen2_moe_57b": "mlp", "mixtral": "block_sparse_moe"}
MOE_WEIGHT_NAME_MAP = {
    **dict.fromkeys(["ds2", "qwen2_moe", "qwen2_moe_57b"], {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}),
    "mixtral": {"gate": "w1", "up": "w3", "down": "w2"},
}
SHARED_NAME = {"ds2": "shared_experts", "qwen2_moe": "shared_expert", "qwen2_moe_57b": "shared_expert"}


def weight_key(model_id: str, layer: int, expert: int | str, block: str) -> str:
    """state_dict key of one linear block; `expert="shared"` names the shared expert(s)  (moe_utils.py:44-60)."""
    mlp, lin = MOE_MLP_NAME_MAP[model_id], MOE_WEIGHT_NAME_MAP[model_id][block]
    if expert == "shared":
        return f"model.layers.{layer}.{mlp}.{SHARED_NAME[model_id]}.{lin}.weight"
    return f"model.layers.{layer}.{mlp}.experts.{expert}.{lin}.weight"


def experts_from_state_dict(state_dict: dict, model_id: str, layer: int, num_experts: int):
    """[(W13 [2I, K] = [gate; up], W2 [K, I])] per routed expert, plus the shared expert (if the family has one) as the last entry."""
    out = []
    names = list(range(num_experts)) + (["shared"] if model_id in SHARED_NAME and weight_key(model_id, layer, "shared", "gate") in state_dict else [])
    for e in names:
        g, u, d = (state_dict[weight_key(model_id, layer, e, b)] for b in ("gate", "up", "down"))
        out.append((torch.cat([g, u], dim=0), d))
    return out


def hadamard_matrix(n: int) -> torch.Tensor:
    """The orthonormal matrix Q of the online rotation, y = Q x with Q = (H_K kron S_{n/K}) / sqrt(n), fp64
    (index p = k * (n/K) + j, mxmoe/quant/hadamard_utils.py:66-81,100-104)."""
    hk, k = get_hadK(n)
    m = n // k
    s = np.array([[1.0]])
    while s.shape[0] < m:
        s = np.block([[s, s], [s, -s]])
    q = np.kron(hk.astype(np.float64), s) if hk is not None else s
    return torch.from_numpy(q / np.sqrt(n))


def rotate_input_weights(w: torch.Tensor) -> torch.Tensor:
    """W [N, n] -> W Q^T (fp64 product, back to W's dtype), so that (W Q^T)(Q x) = W x for the online rotation y = Q x of the
    block's input (rotation.py:353-364 does the same with its Q on the MLP input weights)."""
    q = hadamard_matrix(w.shape[1])
    return (w.to(torch.float64) @ q.T).to(w.dtype)


def recover_grid(w: torch.Tensor, bits: int, gsize: int, sym: bool):
    """Codes, scale and zero point of a weight matrix that is ALREADY on a quantisation grid: every group of `w` [N, K] holds values
    `scale * (q - zero)` with integer q in 0 .. 2^bits - 1 and an integer zero, stored in fp16 or bf16 (what a GPTQ run saves:
    mxmoe/quant/gptq.py:21-25 is the grid, :539-546 the `state_dict` of fake-quantised weights).  Re-quantising such a matrix by
    min / max would move it (its extreme codes need not be in use); this finds the grid itself.
    -> (q [N, K] int, scale, zp) with value = q * scale + zp as `weights.pack_codes` takes them: signed codes and zp = 0 for symmetric
    grids, codes from 0 and zp = (lowest value in use) otherwise.  Raises ValueError for a group that lies on no such grid.

    Per group: the smallest non-zero magnitude is j * scale for a small j (weights cluster around zero, so j = 1 nearly always); for
    j = 1, 2, ... the candidate is refined by least squares, first over the values within 8 steps of zero, then over the whole group
    (a GPTQ scale is an fp32 number, and the stored values carry their type's rounding: an 8-bit code of 127 steps kept in bf16 is off
    by up to half a step, so such a file does not determine its codes and the nearest ones are taken); the first candidate under which
    every value is within 0.3 (plus the type's rounding) of an integer multiple and the integers span at most 2^bits - 1 is taken and
    rounded to fp16, the type the kernels read scales in."""
    n, k = w.shape
    g = k if gsize == -1 else gsize
    v = w.to(torch.float64).reshape(-1, g)
    maxq = (1 << bits) - 1
    # distance from an integer multiple that storage rounding alone explains: half the type's spacing at the largest multiple
    eps = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}.get(w.dtype, 0.0)
    tol = min(0.49, 0.3 + eps * maxq)
    mag = v.abs()
    vmin_nz = torch.where(mag > 0, mag, torch.full_like(mag, float("inf"))).amin(dim=1, keepdim=True)
    flat = ~torch.isfinite(vmin_nz)                                       # all-zero groups: any scale does
    vmin_nz = torch.where(flat, torch.ones_like(vmin_nz), vmin_nz)
    scale = torch.zeros_like(vmin_nz)
    done = torch.zeros_like(flat)
    for j in range(1, 9):
        cand = vmin_nz / j
        t0 = v / cand
        near = t0.abs() <= 8.5                                              # multiples small enough for the first guess to place
        ok = (((t0 - t0.round()).abs() * near).amax(dim=1, keepdim=True) < 0.3)
        ls = lambda t, m: ((v * t * m).sum(dim=1, keepdim=True) / (t * t * m).sum(dim=1, keepdim=True).clamp_min(1e-300))
        s1 = torch.where(flat, torch.ones_like(cand), ls(t0.round(), near))
        s2 = torch.where(flat, torch.ones_like(cand), ls((v / s1).round(), torch.ones_like(near)))
        t2 = v / s2
        ti = t2.round()
        ok &= ((t2 - ti).abs().amax(dim=1, keepdim=True) < tol) & ((ti.amax(dim=1, keepdim=True) - ti.amin(dim=1, keepdim=True)) <= maxq)
        take = ok & ~done
        scale = torch.where(take, s2.to(torch.float16).to(torch.float64), scale)
        done |= ok
    if not bool(done.all()):
        bad = int((~done).nonzero()[0, 0])
        raise ValueError(f"group {bad} (channel {bad // (k // g)}) is not on a {bits}-bit grid")
    t = (v / scale).round()
    if bool(((t * scale - v).abs() > 0.5 * scale).any()):
        raise ValueError("refined scale does not reproduce the stored values")
    if sym:
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        if bool((t.amin() < lo) | (t.amax() > hi)):
            raise ValueError(f"symmetric {bits}-bit codes outside {lo} .. {hi}")
        q, zp = t, torch.zeros_like(scale)
    else:
        tmin = t.amin(dim=1, keepdim=True)
        q, zp = t - tmin, tmin * scale
    return q.reshape(n, k), scale.to(torch.float16), zp.to(torch.float16)


def ingest_fake_quant(w: torch.Tensor, qparams, keep_codes: bool = False) -> PackedWeight:
    """Pack a fake-quantised weight matrix (GPTQ output) without quantising it again.  Symmetric weight-only formats are stored
    offset-binary like their RTN counterparts."""
    a_bits, w_bits, gsize, sym = qparams
    n, k = w.shape
    if w_bits >= 16:
        return PackedWeight(w.to(torch.float16).contiguous(), None, tuple(qparams), n, k)
    q, scale, zp = recover_grid(w, w_bits, gsize, sym)
    return pack_codes(q, scale, zp, tuple(qparams), n, k, keep_codes)


def load_fake_quant_state_dict(path: str) -> dict:
    """The `.pt` file a GPTQ run writes (gptq.py:546: `torch.save(model.state_dict(), ...)`), read as tensors only."""
    return torch.load(path, map_location="cpu", weights_only=True)


def pack_layer(experts, formats, rotate: int = 0, model: str = "", layer: int = 0, num_shared: int = 0, device="cpu", fake_quant: bool = False):
    """experts: [(W13, W2)] fp16 (shared expert last when num_shared > 0); formats: [(gate_up qparams, down qparams)].
    rotate as in the operators: 0 never, 1 blocks with quantised activations, 2 every block.
    fake_quant: the weights are a GPTQ run's fake-quantised output (rotated there already, if at all: gptq.py:525-528), so they are
    neither rotated nor re-quantised here; their grid is recovered (`recover_grid`) and packed; `rotate` is only recorded.
    Returns ({tensor name: tensor}, metadata dict)."""
    tensors, meta_e = {}, []
    for e, ((w13, w2), (gu, dn)) in enumerate(zip(experts, formats)):
        if not fake_quant and (rotate == 2 or (rotate == 1 and gu[0] < 16)):
            w13 = rotate_input_weights(w13)
        if not fake_quant and (rotate == 2 or (rotate == 1 and dn[0] < 16)):
            w2 = rotate_input_weights(w2)
        for name, w, qp in (("w13", w13, gu), ("w2", w2, dn)):
            p = ingest_fake_quant(w.to(device), tuple(qp)) if fake_quant else quantize_and_pack(w.to(device), tuple(qp))
            tensors[f"e{e}.{name}.data"] = p.data.cpu().contiguous()
            if p.scale is not None:
                tensors[f"e{e}.{name}.scale"] = p.scale.cpu().contiguous()
        meta_e.append({"gate_up": list(gu), "down": list(dn), "n13": w13.shape[0], "k13": w13.shape[1], "n2": w2.shape[0], "k2": w2.shape[1]})
    n_routed = len(experts) - (1 if num_shared else 0)
    meta = {"format": FORMAT_VERSION, "model": model, "layer": layer, "num_experts": n_routed, "num_shared": num_shared,
            "hidden": int(experts[0][0].shape[1]), "inter": int(experts[0][1].shape[1]), "rotate": rotate, "experts": meta_e}
    return tensors, meta


def save_layer(path: str, tensors: dict, meta: dict) -> None:
    from safetensors.torch import save_file

    save_file(tensors, path, metadata={"mxmoe_layer": json.dumps(meta)})


def load_layer(path: str, device="cuda"):
    """-> (w13: [PackedWeight], w2: [PackedWeight], metadata).  Tensors are read with safetensors (no code is executed from the file)."""
    from safetensors import safe_open

    with safe_open(path, framework="pt", device=str(device)) as f:
        meta = json.loads(f.metadata()["mxmoe_layer"])
        if meta.get("format") != FORMAT_VERSION:
            raise ValueError(f"{path}: layer file format {meta.get('format')} (this build reads {FORMAT_VERSION})")
        names = set(f.keys())
        w13, w2 = [], []
        for e, em in enumerate(meta["experts"]):
            for dst, name, qp, n, k in ((w13, "w13", em["gate_up"], em["n13"], em["k13"]), (w2, "w2", em["down"], em["n2"], em["k2"])):
                scale = f.get_tensor(f"e{e}.{name}.scale") if f"e{e}.{name}.scale" in names else None
                a_bits, w_bits, gsize, sym = qp
                dst.append(PackedWeight(f.get_tensor(f"e{e}.{name}.data"), scale, (a_bits, w_bits, gsize, bool(sym)), n, k))
    return w13, w2, meta


def formats_from_qconfig(qcfg_layer: dict, num_experts: int, has_shared: bool):
    """One layer of a qconfig JSON ({"experts": {e: {gate, up, down}}}) -> [(gate_up qparams, down qparams)]; gate and up must agree
    (they are one fused GEMM), the shared expert is entry `num_experts` and takes its "gate" format for both blocks, as the workload
    generator does (mxmoe/kernels/gen_workload.py:93-94)."""
    def qp(lin):
        if lin["w_bits"] >= 16 and lin["a_bits"] >= 16:
            return (16, 16, -1, True)
        return (lin["a_bits"], lin["w_bits"], lin["w_gsize"], bool(lin["w_sym"]))

    out = []
    for e in range(num_experts + (1 if has_shared else 0)):
        ex = qcfg_layer["experts"][str(e)] if str(e) in qcfg_layer["experts"] else qcfg_layer["experts"][e]
        if qp(ex["gate"]) != qp(ex["up"]):
            raise ValueError(f"expert {e}: gate and up must share a format")
        out.append((qp(ex["gate"]), qp(ex["gate"] if e == num_experts else ex["down"])))
    return out
