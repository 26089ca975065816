"""Bit-width / tile allocator on the gfx950 kernel profile.

Chooses, per expert and linear block (gate, up, down), one quantisation strategy so that the layer's calibration loss L and its
GroupGEMM run time T (from the kernel-profile table) are traded off under a weight-memory budget: the reference's integer
program (mxmoe/quant/bits_solver.py:201-422) with the same variables, constraints and objective, solved with scipy's HiGHS
(`scipy.optimize.milp`) instead of gurobipy.

    x[e,n,s] in {0,1}            block n of expert e uses strategy s                      (bits_solver.py:316)
    y[e,n,s,t] in {0,1}, sum_t=1 tile combination used for that choice                    (:317, :370-371)
    L = sum x * delta[e][n][s]                                                            (:319-322)
    T = sum x * runtime_cost[e][n][s][t] * y                                              (:323-329)
    minimise L^r * T^(1-r)   (r = 1: loss only, r = 0: time only; else r log L + (1-r) log T)   (:331-356)
    sum wbits[s] * size[e] * x <= budget                                                  (:359-364)
    sum_s x[e,n,s] = 1;  x[e,0,s] = x[e,1,s]  (gate and up share a format)                (:366-367, :377-378)
    --exp_alloc: one strategy per expert (x equal over n)                                 (:277-314)

How the non-linear parts are handled without a non-convex solver:
  * y only appears in T and the y of different (e,n,s) are independent, so the optimal y picks, per (e,n,s), the cheapest tile
    combination: T = sum x * min_t cost (`tile_mode="per_block"`, the program as written).  A fused kernel is generated from ONE
    tile combination per layer; `tile_mode="per_layer"` therefore also solves the program once per combination t with
    T = sum x * cost[..][t] and keeps the best; the exported tile configuration is that combination.
  * L^r T^(1-r) is increasing in both L and T, so its minimum is a Pareto point of (L, T).  Pareto points are produced by the
    minimum over the convex hull of the front is found by iterating the weight of a weighted sum L + lam T; from that point the
    front is walked in both directions with epsilon-constraint steps (minimise L subject to T <= tau, then minimise T subject to
    L <= that L) until a bound shows that no further point can win.  Every candidate is an exact MILP optimum.
"""
from __future__ import annotations

import argparse
import itertools
import json
import math
import os
from collections import defaultdict

import numpy as np

from .kernels.qconfig import QLinearConfig
from .perf_table import ProblemShape, get_runtime_cost

WEIGHT_IDX_2_NAME = {0: "gate", 1: "up", 2: "down"}


def value_to_prob(freq):
    """bits_solver.py:20-22."""
    total = sum(freq)
    return [f / total for f in freq]


def get_strategy_bits(qcfg: str):
    """(weight bits incl. group metadata, activation bits) of a strategy string  (bits_solver.py:581-597)."""
    table = {
        "w8a16_g-1": (8, 16), "w4a16_g-1": (4, 16), "w4a16_g128": (4.25, 16), "w3a16_g128": (3.25, 16), "w2a16_g128": (2.25, 16),
        "w1a16_g128": (1.25, 16), "w4a4_g-1": (4, 4), "w8a8_g-1": (8, 8), "w4a4_g128": (4.25, 4.25),
    }
    for k, v in table.items():
        if k in qcfg:
            return v
    raise ValueError(f"unknown strategy {qcfg}")


def get_num_weights(model_id: str, num_layers: int):
    """(weight matrices in the model, per layer), shared experts counted by their width  (bits_solver.py:646-654)."""
    per_layer = {"qwen2_moe": (60 + 4) * 3, "qwen2_moe_57b": (64 + 8) * 3, "mixtral": 8 * 3, "ds2": (64 + 2) * 3}[model_id]
    return num_layers * per_layer, per_layer


def parse_strategy(qname: str) -> dict:
    """"w4a4_g-1_sym" -> QLinearConfig dict  (bits_solver.py:32-37)."""
    head, g, s = qname.split("_")[:3]
    w_bits, a_bits = (int(v) for v in head.split("w")[1].split("a"))
    gsize, sym = int(g[1:]), s == "sym"
    return QLinearConfig(w_bits=w_bits, w_gsize=gsize, w_sym=sym, a_bits=a_bits, a_gsize=gsize, a_sym=sym).to_dict()


def export_qconfig(select_strategies, save_path: str | None = None):
    """(strategies per layer / expert / block, tile configuration per layer) -> qconfig JSON + `<name>_tile_cfg.json`
    (bits_solver.py:25-71: same file names and shapes; tile configurations are written as `repr` strings)."""
    if save_path is not None and not save_path.endswith(".json"):
        raise ValueError("Invalid save_path, must be a json file.")
    select, tiled = select_strategies
    select = dict(select)
    tiled = {k: repr(v) for k, v in tiled.items()}
    lt = select.pop("LT", None)
    model_qcfg = {
        layer: {"experts": {e: {WEIGHT_IDX_2_NAME[n]: parse_strategy(q) for n, q in ecfg.items()} for e, ecfg in lcfg.items()}}
        for layer, lcfg in select.items()
    }
    if save_path is not None:
        os.makedirs(os.path.dirname(save_path) or ".", exist_ok=True)
        cur = dict(model_qcfg)
        if lt is not None:
            cur["LT"] = lt
        with open(save_path, "w") as f:
            json.dump(cur, f)
        with open(f"{save_path.split('.json')[0]}_tile_cfg.json", "w") as f:
            json.dump(tiled, f)
    return model_qcfg


def build_workloads(model_id: str, batch_range: int, offline_stats: dict, num_layers: int):
    """Per layer: [expert][block] problem shapes at `batch_range` tokens, access probabilities, relative expert sizes
    (bits_solver.py:545-578; the shared experts form one extra expert of width N * num_shared that sees every token)."""
    n_sh = offline_stats["num_shared_experts"]
    scale = batch_range / offline_stats["num_tokens"]
    N, K = offline_stats["NK"]
    workloads, sizes, freqs = [], [], []
    for layer in range(num_layers):
        if model_id == "ds2" and layer == 0:  # dense first layer (bits_solver.py:561-565)
            workloads.append([[ProblemShape(batch_range, 10944, 2048), ProblemShape(batch_range, 10944, 2048), ProblemShape(batch_range, 2048, 10944)]])
            sizes.append([1])
            freqs.append([1])
            continue
        layer_freq = offline_stats[f"layer-{layer}"]["access_freq"]
        ms = [int(scale * v) for v in layer_freq] + ([batch_range] if n_sh else [])
        ns = [N] * len(layer_freq) + ([N * n_sh] if n_sh else [])
        workloads.append([[ProblemShape(m, n, K), ProblemShape(m, n, K), ProblemShape(m, K, n)] for m, n in zip(ms, ns)])
        sizes.append([(n * K) / (N * K) for n in ns])
        freqs.append(value_to_prob(ms))
    return workloads, freqs, sizes


# ---------------------------------------------------------------------------------------------------------------------------------
# one layer
# ---------------------------------------------------------------------------------------------------------------------------------
class LayerProgram:
    """The layer-level program for fixed loss and time coefficients (both [E][N][S])."""

    def __init__(self, delta, tcost, wbits, sizes, budget, exp_alloc: bool = False):
        self.delta = np.asarray(delta, dtype=np.float64)
        self.tcost = np.asarray(tcost, dtype=np.float64)
        self.E, self.N, self.S = self.delta.shape
        assert self.tcost.shape == self.delta.shape
        E, N, S = self.E, self.N, self.S
        self.nv = E * N * S
        rows, lo, hi = [], [], []

        def row(entries, lb, ub):
            r = np.zeros(self.nv)
            for idx, v in entries:
                r[idx] += v
            rows.append(r)
            lo.append(lb)
            hi.append(ub)

        for e, n in itertools.product(range(E), range(N)):          # one strategy per block
            row([(self.idx(e, n, s), 1.0) for s in range(S)], 1.0, 1.0)
        if N >= 2:
            for e, s in itertools.product(range(E), range(S)):      # gate and up share a strategy
                row([(self.idx(e, 0, s), 1.0), (self.idx(e, 1, s), -1.0)], 0.0, 0.0)
        if exp_alloc:
            for e, s, n in itertools.product(range(E), range(S), range(2, N)):
                row([(self.idx(e, 0, s), 1.0), (self.idx(e, n, s), -1.0)], 0.0, 0.0)
        row([(self.idx(e, n, s), wbits[s] * sizes[e]) for e, n, s in itertools.product(range(E), range(N), range(S))], -np.inf, float(budget))
        self.A, self.lo, self.hi = np.array(rows), np.array(lo), np.array(hi)
        self.cL, self.cT = self.delta.reshape(-1), self.tcost.reshape(-1)

    def idx(self, e, n, s):
        return (e * self.N + n) * self.S + s

    def solve(self, c, extra=None):
        """min c.x over the feasible set, optionally with extra rows [(coeffs, ub)]; returns x (0/1 array) or None."""
        from scipy.optimize import Bounds, LinearConstraint, milp

        A, lo, hi = self.A, self.lo, self.hi
        if extra:
            A = np.vstack([A] + [r[None, :] for r, _ in extra])
            lo = np.concatenate([lo, [-np.inf] * len(extra)])
            hi = np.concatenate([hi, [ub for _, ub in extra]])
        res = milp(c, constraints=LinearConstraint(A, lo, hi), integrality=np.ones(self.nv), bounds=Bounds(0, 1), options={"mip_rel_gap": 0.0})
        if res.x is None:
            return None
        return np.rint(res.x)

    def LT(self, x):
        return float(self.cL @ x), float(self.cT @ x)

    def pareto_point(self, tau):
        """The Pareto point with the smallest loss among those with T <= tau (loss first, then time)."""
        x = self.solve(self.cL, [(self.cT, tau)])
        if x is None:
            return None
        L = self.cL @ x
        x2 = self.solve(self.cT, [(self.cL, L * (1 + 1e-12) + 1e-12)])
        return x2 if x2 is not None else x

    def optimise(self, r: float, max_points: int = 16):
        """argmin L^r T^(1-r).  Returns (x, L, T)."""
        if r >= 1.0:
            x = self.solve(self.cL)
            if x is None:
                raise ValueError("memory budget cannot be met by any assignment")
            x2 = self.solve(self.cT, [(self.cL, self.cL @ x * (1 + 1e-12) + 1e-12)])  # ties in loss: the faster one
            x = x2 if x2 is not None else x
            return (x, *self.LT(x))
        x_t = self.solve(self.cT)
        if x_t is None:
            raise ValueError("memory budget cannot be met by any assignment")
        x2 = self.solve(self.cL, [(self.cT, self.cT @ x_t * (1 + 1e-12) + 1e-12)])  # ties in time: the one with less loss
        x_t = x2 if x2 is not None else x_t
        if r <= 0.0:
            return (x_t, *self.LT(x_t))
        x_l = self.optimise(1.0)[0]
        (l_hi, t_lo), (l_lo, t_hi) = self.LT(x_t), self.LT(x_l)
        step = 1 - 1e-5  # well outside the solver's feasibility tolerance: a point must not come back as its own successor

        def score_lt(L, T):
            return r * math.log(max(L, 1e-300)) + (1 - r) * math.log(max(T, 1e-300))

        def score(x):
            return score_lt(*self.LT(x))

        best = min((x_t, x_l), key=score)
        # 1. supported Pareto points: at a minimiser of r log L + (1-r) log T over the convex hull of the front the weighted sum
        #    L + lam T is minimal for lam = (1-r)/r * L/T; iterate that fixed point
        lam = (1 - r) / r * l_lo / t_hi
        seen = set()
        for _ in range(24):
            x = self.solve(self.cL + lam * self.cT)
            if x is None:
                break
            L, T = self.LT(x)
            if score(x) < score(best):
                best = x
            key = (round(L, 9), round(T, 9))
            if key in seen:
                break
            seen.add(key)
            lam = (1 - r) / r * L / T
        # 2. the points between supported ones: walk the front from there in both directions (epsilon-constraint steps); a direction
        #    ends when even the best conceivable remaining point (its own L with the smallest T, or its T with the smallest L)
        #    cannot beat the incumbent, so the result is exact unless a walk is cut off after `max_points` steps
        start = best
        x = start
        for _ in range(max_points):  # towards smaller T / larger L
            x = self.pareto_point(self.cT @ x * step)
            if x is None:
                break
            if score(x) < score(best):
                best = x
            if score_lt(self.LT(x)[0], t_lo) >= score(best):
                break
        x = start
        for _ in range(max_points):  # towards smaller L / larger T
            xn = self.solve(self.cT, [(self.cL, self.cL @ x * step)])
            if xn is None:
                break
            x = self.pareto_point(self.cT @ xn * (1 + 1e-9))
            if x is None:
                break
            if score(x) < score(best):
                best = x
            if score_lt(l_lo, self.LT(x)[1]) >= score(best):
                break
        return (best, *self.LT(best))


def solve_layer(strategies, delta, runtime_cost, wbits, sizes, budget, r: float, exp_alloc: bool = False, tile_mode: str = "per_layer"):
    """One layer of the program.  delta[e][n][s], runtime_cost[e][n][s][t] (t = tile combination).
    Returns ({e: {n: strategy}}, (L, T), index of the tile combination a fused kernel should be generated from)."""
    cost = np.asarray(runtime_cost, dtype=np.float64)
    E, N, S, Tn = cost.shape
    if r >= 1.0:
        cost = np.ones_like(cost)  # the reference drops the time term altogether (bits_solver.py:256-259)
    per_block = cost.min(axis=3)
    best = None
    if tile_mode == "per_block":
        prog = LayerProgram(delta, per_block, wbits, sizes, budget, exp_alloc)
        x, L, T = prog.optimise(r)
        xs = x.reshape(E, N, S)
        t_star = int(np.argmin([(xs * cost[..., t]).sum() for t in range(Tn)]))
        best = (xs, L, T, t_star)
    elif tile_mode == "per_layer":
        for t in range(Tn):
            prog = LayerProgram(delta, cost[..., t], wbits, sizes, budget, exp_alloc)
            x, L, T = prog.optimise(r)
            val = r * math.log(max(L, 1e-300)) + (1 - r) * math.log(max(T, 1e-300))
            if best is None or val < best[4]:
                best = (x.reshape(E, N, S), L, T, t, val)
    else:
        raise ValueError(f"tile_mode {tile_mode!r}")
    xs, L, T, t_star = best[:4]
    chosen = defaultdict(dict)
    for e, n in itertools.product(range(E), range(N)):
        chosen[e][n] = strategies[int(np.argmax(xs[e, n]))]
    return dict(chosen), (L, T), t_star


def convert_to_delta_array(strategies, strategy_loss, layer_idx, num_experts: int, num_blocks: int = 3):
    """delta[e][n][s] from {strategy: {layer: {expert: [gate, up, down]}}}  (bits_solver.py:228-236)."""
    return [[[strategy_loss[s][str(layer_idx)][str(e)][n] for s in strategies] for n in range(num_blocks)] for e in range(num_experts)]


def solve_model_qconfig_layer_level(model_id, strategies, strategy_loss, strategy_wbits, layer_wbits_budget, workloads, expert_sizes,
                                    performance_table, r: float, exp_alloc: bool = False, tile_mode: str = "per_layer", tile_cfgs=None,
                                    verbose: bool = True):
    """Layer by layer (bits_solver.py:201-422).  Returns ({"LT": {layer: (L, T)}, layer: {expert: {block: strategy}}},
    {layer: tuple of TileConfig})."""
    num_layers = len(next(iter(strategy_loss.values())))
    qconfig, tilecfg = {"LT": {}}, {}
    for layer in range(num_layers):
        if model_id == "ds2" and layer == 0:  # dense layer: fixed (bits_solver.py:243-247)
            qconfig["LT"][layer] = [0, 0]
            qconfig[layer] = {0: {0: "w4a4_g-1_asym", 1: "w4a4_g-1_asym", 2: "w4a4_g-1_asym"}}
            tilecfg[layer] = []
            continue
        E = len(expert_sizes[layer])
        combos, cost = get_runtime_cost(workloads[layer], strategies, performance_table, tile_cfgs)
        delta = convert_to_delta_array(strategies, strategy_loss, layer, E)
        chosen, lt, t_star = solve_layer(strategies, delta, cost, strategy_wbits, expert_sizes[layer], layer_wbits_budget, r, exp_alloc, tile_mode)
        qconfig["LT"][layer] = lt
        qconfig[layer] = chosen
        tilecfg[layer] = combos[t_star]
        if verbose:
            hist = defaultdict(int)
            for e in chosen.values():
                for q in e.values():
                    hist[q] += 1
            print(f"layer {layer}: L {lt[0]:.4f}  T {lt[1]:.4f}  {dict(hist)}")
    return qconfig, tilecfg


def solve_model_qconfig_model_level(strategies, strategy_loss, strategy_wbits, model_wbits_budget):
    """Whole model at once, loss only: min sum x * loss  s.t. sum wbits * x <= budget, one strategy per block
    (bits_solver.py:119-198).  Returns {layer: {expert: {block: strategy}}}."""
    from scipy.optimize import Bounds, LinearConstraint, milp

    num_layers = len(next(iter(strategy_loss.values())))
    E = len(next(iter(strategy_loss.values()))["0"])
    N, S = 3, len(strategies)
    keys = list(itertools.product(range(num_layers), range(E), range(N)))
    c = np.array([strategy_loss[strategies[s]][str(l)][str(e)][n] for (l, e, n) in keys for s in range(S)])
    nv = len(c)
    A = np.zeros((len(keys) + 1, nv))
    for i in range(len(keys)):
        A[i, i * S:(i + 1) * S] = 1.0
    A[-1] = np.tile(np.asarray(strategy_wbits, dtype=np.float64), len(keys))
    lo = np.concatenate([np.ones(len(keys)), [-np.inf]])
    hi = np.concatenate([np.ones(len(keys)), [float(model_wbits_budget)]])
    res = milp(c, constraints=LinearConstraint(A, lo, hi), integrality=np.ones(nv), bounds=Bounds(0, 1), options={"mip_rel_gap": 0.0})
    if res.x is None:
        raise ValueError("memory budget cannot be met by any assignment")
    x = np.rint(res.x).reshape(len(keys), S)
    out = {l: defaultdict(dict) for l in range(num_layers)}
    for (l, e, n), row in zip(keys, x):
        out[l][e][n] = strategies[int(np.argmax(row))]
    return {l: dict(v) for l, v in out.items()}


def solve_model_qconfig(model_id, strategy_loss, solve_mode, wbits_budget, batch_range, offline_stats, r, exp_alloc=False,
                        tile_mode="per_layer", tile_cfgs=None, verbose=True):
    """bits_solver.py:600-643."""
    strategies = sorted(strategy_loss)
    wbits = [get_strategy_bits(s)[0] for s in strategies]
    num_layers = len(next(iter(strategy_loss.values())))
    if solve_mode == "model":
        return solve_model_qconfig_model_level(strategies, strategy_loss, wbits, wbits_budget), {}
    workloads, _, sizes = build_workloads(model_id, batch_range, offline_stats, num_layers)
    return solve_model_qconfig_layer_level(model_id, strategies, strategy_loss, wbits, wbits_budget, workloads, sizes,
                                           offline_stats["performance_table"], r, exp_alloc, tile_mode, tile_cfgs, verbose)


def get_offline_stats(trace_file: str, perf_file: str) -> dict:
    """Gate trace + kernel profile in one dict  (bits_solver.py:657-664)."""
    with open(trace_file) as f:
        trace = json.load(f)
    with open(perf_file) as f:
        trace["performance_table"] = json.load(f)
    return trace


def get_strategy_loss(calib_loss_list: dict, filter_list) -> dict:
    """{strategy: path of {layer: {expert: [gate, up, down]}} JSON} -> losses of the strategies in `filter_list`
    (bits_solver.py:85-97)."""
    out = {}
    for qname, path in calib_loss_list.items():
        if filter_list and not any(f in qname for f in filter_list):
            continue
        with open(path) as f:
            out[qname] = json.load(f)
    return out


def synthetic_strategy_loss(cfg, strategies, layer: int = 0) -> dict:
    """A calibration-free stand-in for the reference's per-block calibration losses (which need the real checkpoints): for
    y = W x with x ~ N(0, I), E|W_q x_q - W x|^2 ~ |W_q - W|_F^2 + |W|_F^2 * eps_a, where eps_a is the relative squared error of the
    strategy's activation quantiser on Gaussian rows; weighted by how often the expert is used.  Same shape as the loss files:
    {strategy: {layer: {expert: [gate, up, down]}}}."""
    import torch

    from . import synth
    from .kernels.tile_config import get_info_from_qcfg_str
    from .quant import Quantizer

    ids, _ = synth.make_routing(cfg)
    freq = torch.bincount(ids.reshape(-1).to(torch.int64), minlength=cfg.num_experts).double()
    prob = (freq / freq.sum()).tolist() + ([1.0] if cfg.num_shared else [])
    g = torch.Generator().manual_seed(5)
    out = {s: {str(layer): {}} for s in strategies}
    eps_a = {}
    for s in strategies:
        w_bits, a_bits, gsize, sym = get_info_from_qcfg_str(s)
        if a_bits >= 16:
            eps_a[s] = {k: 0.0 for k in (cfg.hidden, cfg.inter)}
        else:
            eps_a[s] = {}
            for k in (cfg.hidden, cfg.inter):
                x = torch.randn(64, k, generator=g).half()
                xq = Quantizer(a_bits, True, -1).fake_quant(x)
                eps_a[s][k] = float(((xq.float() - x.float()) ** 2).sum() / (x.float() ** 2).sum())
    for e in range(len(prob)):
        w13, w2 = synth.expert_weights(cfg, e)
        i = w13.shape[0] // 2
        blocks = (w13[:i], w13[i:], w2)
        for s in strategies:
            w_bits, a_bits, gsize, sym = get_info_from_qcfg_str(s)
            vals = []
            for w in blocks:
                wq = Quantizer(w_bits, sym, gsize).fake_quant(w)
                wf = w.float()
                vals.append(prob[e] * float(((wq.float() - wf) ** 2).sum() + (wf ** 2).sum() * eps_a[s][w.shape[1]]))
            out[s][str(layer)][str(e)] = vals
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Allocate bit-widths and tiles per expert block on the gfx950 kernel profile")
    ap.add_argument("--model", default="qwen2_moe", choices=["qwen2_moe", "ds2", "mixtral", "qwen2_moe_57b"])
    ap.add_argument("--synthetic", default=None, metavar="CONFIG",
                    help="one of the synthetic workloads (c2, c3, ...): routing trace and loss stand-ins are made from its seeded data")
    ap.add_argument("--strategies", nargs="+", default=["w4a4_g-1_sym", "w8a8_g-1_sym"], help="candidate strategies with --synthetic")
    ap.add_argument("--loss", nargs="+", default=[], metavar="STRATEGY=FILE",
                    help="calibration loss files, one per strategy: JSON {layer: {expert: [gate, up, down]}}")
    ap.add_argument("--batch", type=int, default=512, help="tokens per step the run time is estimated for")
    ap.add_argument("--wbits", type=float, required=True, help="average weight bits per parameter")
    ap.add_argument("--tokens", type=int, default=None, help="tokens of the synthetic workload (default: the workload's own)")
    ap.add_argument("--solve_mode", choices=["layer", "model"], default="layer")
    ap.add_argument("--filter_list", nargs="+", default=[])
    ap.add_argument("--r", type=float, default=-1, help="weight of the loss in the objective; -1 sweeps 0, 0.25, 0.5, 0.75, 1")
    ap.add_argument("--trace_file", default=None, help="expert activation frequency trace (moe-gate.json)")
    ap.add_argument("--perf_file", default="perf/performance_table.json")
    ap.add_argument("--exp_alloc", action="store_true", help="one strategy per expert instead of per linear block")
    ap.add_argument("--tile_mode", choices=["per_layer", "per_block"], default="per_layer")
    ap.add_argument("--out_dir", default="qconfigs")
    a = ap.parse_args(argv)
    if a.synthetic:
        from . import synth

        cfg = synth.get_config(a.synthetic, a.tokens)
        strategy_loss = synthetic_strategy_loss(cfg, sorted(a.strategies))
        stats = synth.trace_dict(cfg)
        with open(a.perf_file) as f:
            stats["performance_table"] = json.load(f)
        a.batch = cfg.tokens
        synthetic_layer_n = 3 * (cfg.num_experts + cfg.num_shared)
    else:
        synthetic_layer_n = None
        if not a.loss or not a.trace_file:
            ap.error("--loss and --trace_file are required without --synthetic")
        strategy_loss = get_strategy_loss(dict(item.split("=", 1) for item in a.loss), a.filter_list)
        stats = get_offline_stats(a.trace_file, a.perf_file)
    num_layers = len(next(iter(strategy_loss.values())))
    model_n, layer_n = get_num_weights(a.model, num_layers)
    if synthetic_layer_n is not None:  # the synthetic layer's own expert count (some workloads leave the shared experts out)
        model_n, layer_n = num_layers * synthetic_layer_n, synthetic_layer_n
    budget = a.wbits * (model_n if a.solve_mode == "model" else layer_n)
    mxdir = "+".join(sorted(strategy_loss))
    for r in ([0.0, 0.25, 0.5, 0.75, 1.0] if a.r == -1 else [a.r]):
        sel = solve_model_qconfig(a.model, strategy_loss, a.solve_mode, budget, a.batch, stats, r, a.exp_alloc, a.tile_mode)
        suffix = "_exp_alloc" if a.exp_alloc else ""
        path = f"{a.out_dir}/{mxdir}/{a.model}_S{a.solve_mode}_bs{a.batch}_wbits{a.wbits}_r{r}{suffix}.json"
        export_qconfig(sel, path)
        print(f"wrote {path}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
