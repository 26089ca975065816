"""Bit-width / tile allocator: the HiGHS solution against exhaustive enumeration on small layers, and the file formats it writes."""
import itertools
import json
import math

import numpy as np
import pytest

from mxmoe_amd import bits_solver as B
from mxmoe_amd.kernels.qconfig import build_qmodel_cfg_from_json


def _brute(delta, cost, wbits, sizes, budget, r, exp_alloc, tile_mode):
    """Every assignment with gate == up (and one strategy per expert under exp_alloc); objective r log L + (1-r) log T."""
    delta, cost = np.asarray(delta), np.asarray(cost)
    E, N, S, Tn = cost.shape
    if r >= 1.0:
        cost = np.ones_like(cost)
    per_expert = [(g, g, d) for g in range(S) for d in range(S) if not exp_alloc or g == d]
    best = None
    for assign in itertools.product(per_expert, repeat=E):
        if sum(wbits[s] * sizes[e] for e, a in enumerate(assign) for s in a) > budget + 1e-9:
            continue
        L = sum(delta[e][n][s] for e, a in enumerate(assign) for n, s in enumerate(a))
        per_t = [sum(cost[e][n][s][t] for e, a in enumerate(assign) for n, s in enumerate(a)) for t in range(Tn)]
        T = min(per_t) if tile_mode == "per_layer" else sum(min(cost[e][n][s]) for e, a in enumerate(assign) for n, s in enumerate(a))
        val = L if r >= 1.0 else (T if r <= 0.0 else r * math.log(L) + (1 - r) * math.log(T))
        if best is None or val < best[0] - 1e-12:
            best = (val, L, T, assign)
    return best


@pytest.mark.parametrize("seed", [0, 1, 2])
@pytest.mark.parametrize("r", [0.0, 0.25, 0.5, 0.75, 1.0])
@pytest.mark.parametrize("exp_alloc,tile_mode", [(False, "per_layer"), (False, "per_block"), (True, "per_layer")])
def test_layer_program_matches_enumeration(seed, r, exp_alloc, tile_mode):
    rng = np.random.default_rng(seed)
    E, N, S, Tn = 3, 3, 3, 2
    strategies = ["w4a4_g-1_sym", "w8a8_g-1_sym", "w4a16_g128_asym"]
    wbits = [B.get_strategy_bits(s)[0] for s in strategies]
    # losses fall and run times rise with the bit-width, with noise: a real trade-off
    delta = rng.uniform(0.5, 1.5, (E, N, S)) * np.array([4.0, 1.0, 2.0])
    cost = rng.uniform(0.5, 1.5, (E, N, S, Tn)) * np.array([1.0, 2.0, 3.0])[None, None, :, None]
    sizes = [1.0, 1.0, 2.0]
    budget = 5.5 * sum(sizes) * N
    want = _brute(delta, cost, wbits, sizes, budget, r, exp_alloc, tile_mode)
    chosen, (L, T), t_star = B.solve_layer(strategies, delta, cost, wbits, sizes, budget, r, exp_alloc, tile_mode)
    assert all(chosen[e][0] == chosen[e][1] for e in range(E))
    if exp_alloc:
        assert all(chosen[e][0] == chosen[e][2] for e in range(E))
    used = sum(wbits[strategies.index(chosen[e][n])] * sizes[e] for e in range(E) for n in range(N))
    assert used <= budget + 1e-9
    got = L if r >= 1.0 else (T if r <= 0.0 else r * math.log(L) + (1 - r) * math.log(T))
    assert got == pytest.approx(want[0], rel=1e-9, abs=1e-9), (chosen, want)
    assert 0 <= t_star < Tn


def test_budget_forces_low_bits_and_infeasible_budget_raises():
    strategies = ["w4a4_g-1_sym", "w8a8_g-1_sym"]
    delta = [[[5.0, 1.0]] * 3] * 2                     # 8 bits always better
    cost = [[[[1.0], [1.0]]] * 3] * 2
    chosen, _, _ = B.solve_layer(strategies, delta, cost, [4, 8], [1, 1], 8 * 6, 1.0)
    assert all(q == "w8a8_g-1_sym" for e in chosen.values() for q in e.values())
    chosen, _, _ = B.solve_layer(strategies, delta, cost, [4, 8], [1, 1], 4 * 6, 1.0)
    assert all(q == "w4a4_g-1_sym" for e in chosen.values() for q in e.values())
    # room for exactly one expert's down block at 8 bits (gate and up move together and would need 8 more)
    chosen, _, _ = B.solve_layer(strategies, delta, cost, [4, 8], [1, 1], 4 * 6 + 4, 1.0)
    assert sorted(q for e in chosen.values() for q in e.values()).count("w8a8_g-1_sym") == 1
    with pytest.raises(ValueError, match="budget"):
        B.solve_layer(strategies, delta, cost, [4, 8], [1, 1], 4 * 6 - 1, 1.0)


def test_model_level_is_a_knapsack():
    strategies = ["w4a4_g-1_sym", "w8a8_g-1_sym"]
    rng = np.random.default_rng(3)
    L, E = 2, 3
    loss = {s: {str(l): {str(e): list(rng.uniform(1, 2, 3) * (3.0 if "w4" in s else 1.0)) for e in range(E)} for l in range(L)} for s in strategies}
    budget = 4 * L * E * 3 + 4 * 5                      # five blocks may take 8 bits
    sel = B.solve_model_qconfig_model_level(strategies, loss, [4, 8], budget)
    gains = sorted((loss[strategies[0]][str(l)][str(e)][n] - loss[strategies[1]][str(l)][str(e)][n], l, e, n) for l in range(L) for e in range(E) for n in range(3))
    top5 = {(l, e, n) for _, l, e, n in gains[-5:]}
    got = {(l, e, n) for l in sel for e in sel[l] for n in sel[l][e] if sel[l][e][n] == "w8a8_g-1_sym"}
    assert got == top5


def test_strategy_bits_and_parse():
    assert B.get_strategy_bits("w4a16_g128_asym") == (4.25, 16) and B.get_strategy_bits("w8a8_g-1_sym") == (8, 8)
    d = B.parse_strategy("w3a16_g128_asym")
    assert (d["w_bits"], d["a_bits"], d["w_gsize"], d["w_sym"]) == (3, 16, 128, False)
    assert B.get_num_weights("qwen2_moe", 24) == (24 * 64 * 3, 64 * 3)
    assert B.value_to_prob([1, 3]) == [0.25, 0.75]


def test_qwen_layer_on_the_gfx950_table(tmp_path):
    """A whole Qwen1.5-MoE layer (60 experts + the shared one) on the regenerated kernel profile: the result honours the budget, is
    written in the reference's qconfig format and feeds the GroupGEMM driver's readers."""
    from mxmoe_amd import synth

    from run_mxmoe_gg import get_qcfg_list

    cfg = synth.get_config("c3")
    trace = synth.trace_dict(cfg)
    trace["NK"] = [cfg.inter, cfg.hidden]
    trace["num_shared_experts"] = 4
    table = json.load(open("perf/performance_table.json"))
    strategies = ["w4a4_g-1_sym", "w8a8_g-1_sym"]
    rng = np.random.default_rng(0)
    E = cfg.num_experts + 1
    loss = {s: {"0": {str(e): list(rng.uniform(0.5, 1.5, 3) * (4.0 if "w4" in s else 1.0)) for e in range(E)}} for s in strategies}
    stats = dict(trace, performance_table=table)
    _, layer_n = B.get_num_weights("qwen2_moe", 1)
    from mxmoe_amd.kernels.tile_config import QCFG_MAP, get_possible_tile_list

    # two candidate tiles per strategy, as the reference hand-picks them (bits_solver.py:426-515)
    tile_cfgs = {q: [t.set_qcfg(QCFG_MAP[q]) for t in get_possible_tile_list("gfx950", q)[:2]] for q in strategies}
    results = {}
    for r in (0.0, 0.5, 1.0):
        sel, tiles = B.solve_model_qconfig("qwen2_moe", loss, "layer", 6.0 * layer_n, 8192, stats, r, tile_cfgs=tile_cfgs, verbose=False)
        results[r] = sel["LT"][0]
        q = sel[0]
        assert len(q) == E and all(q[e][0] == q[e][1] for e in q)
        sizes = [1.0] * cfg.num_experts + [4.0]
        used = sum(B.get_strategy_bits(q[e][n])[0] * sizes[e] for e in q for n in q[e])
        assert used <= 6.0 * layer_n + 1e-9
        assert len(tiles[0]) == len(strategies)
    # more weight on the loss never raises the loss, more weight on time never raises the time
    assert results[1.0][0] <= results[0.5][0] + 1e-9 <= results[0.0][0] + 2e-9
    assert results[0.0][1] <= results[0.5][1] + 1e-9
    path = tmp_path / "qwen2_moe_Slayer_bs8192_wbits6.0_r1.0.json"
    B.export_qconfig((sel, tiles), str(path))
    model = build_qmodel_cfg_from_json(str(path))
    assert len(model.layers["0"].experts) == E
    assert set(get_qcfg_list(str(path), 0)) <= set(strategies)
    tile_json = json.load(open(str(path).replace(".json", "_tile_cfg.json")))
    assert "TileConfig" in tile_json["0"] or "BM" in tile_json["0"]
