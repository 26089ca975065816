"""Host logic mirrored from the reference's Python side: qconfig schema, tile descriptors, workload generation, the
kernel generator and the run_mxmoe_gg helpers.  No GPU."""
import json
import re
from pathlib import Path

import pytest

from mxmoe_amd import synth
from mxmoe_amd.kernels import gen_workload, qconfig, tile_config
from mxmoe_amd.kernels.compose_kernel import KernelType, TemplateGenerator

REF_TABLE = Path("/root/reference/perf/performance_table.json")


def test_qconfig_schema_roundtrip(tmp_path):
    d = synth.qconfig_dict(synth.get_config("c3"))
    d["LT"] = {"note": "popped by readers"}                                # run_mxmoe_gg.py:14, qconfig.py:70
    p = tmp_path / "q-wbits5.00.json"
    p.write_text(json.dumps(d))
    m = qconfig.build_qmodel_cfg_from_json(str(p))
    assert set(m.layers) == {"0"} and len(m.layers["0"].experts) == 60
    e0 = m.layers["0"].experts["0"]
    assert e0.gate == e0.up                                                # gate and up share a format
    assert str(e0.gate) in ("W4A4_g-1_sym", "W8A8_g-1_sym")
    assert e0.gate.qparams() in (synth.W4A4, synth.W8A8)
    assert qconfig.QLinearConfig.from_dict(e0.gate.to_dict()) == e0.gate
    assert set(map(tuple, qconfig.get_all_wbits(m))) == {(4, -1, True), (8, -1, True)}
    uni = qconfig.build_uni_qmodel_cfg(qconfig.QLinearConfig(w_bits=4, a_bits=4, w_sym=True), 2, 3)
    assert len(uni.layers) == 2 and len(uni.layers["1"].experts) == 3


def test_tile_config_repr_is_the_profile_table_key_shape():
    t = tile_config.get_possible_tile_list("gfx950", "w4a4_g-1_sym")[0]
    r = repr(t)
    assert r.startswith("TileConfig(BM=128, BN=256, BK=128, WM=1, WN=4, WK=1, STAGE=3, SPLITK=-1, MMA='MFMA_I32_32x32x32_I8_FROM_I4', QCFGA=QConfig(T_PACK='half', QBITS=4")
    if REF_TABLE.exists():                                                 # same field order as the keys of the reference's table
        ref_key = next(iter(json.loads(REF_TABLE.read_text())["w4a4_g-1_sym"]["3"]))
        assert re.findall(r"(\w+)=", ref_key) == re.findall(r"(\w+)=", r)
    assert t.num_warps == 4 and t.smem_bytes_tile() == 4 * 64 * (64 * 2 + 8)   # activations only (3 x 8 KB) < epilogue patch
    assert tile_config.get_info_from_qcfg_str("w3a16_g128_asym") == (3, 16, 128, False)
    with pytest.raises(ValueError):
        tile_config.TileConfig(BM=128, BN=256, BK=64, WM=2, WN=4, MMA="MFMA_I32_32x32x32_I8").validate()   # 8 waves
    with pytest.raises(ValueError):
        tile_config.get_possible_tile_list("89", "fp16")


def test_tile_config_json_both_forms():
    qs = ["w4a4_g-1_sym", "w8a8_g-1_sym"]
    a = tile_config.load_tile_configs({"w4a4_g-1_sym": [{"BM": 64, "BN": 256, "BK": 128, "WM": 1, "WN": 4}], "w8a8_g-1_sym": [{"BM": 128, "BN": 256, "BK": 64}]}, qs)
    assert a["w4a4_g-1_sym"][0].cpp_type() == "WxAxTile<Op::I4, 64, 256>"
    assert a["w8a8_g-1_sym"][0].QCFGA.QBITS == 8
    pair = (tile_config.get_possible_tile_list("gfx950", qs[0])[1], tile_config.get_possible_tile_list("gfx950", qs[1])[0])
    b = tile_config.load_tile_configs({"11": repr(pair)}, qs)              # the form bits_solver.export_qconfig writes
    assert b[qs[0]][0] == pair[0] and b[qs[1]][0] == pair[1]


def test_gen_workload_follows_the_reference_rules(tmp_path):
    cfg = synth.get_config("c4")
    trace, qcfg = tmp_path / "moe-gate.json", tmp_path / "q-wbits4.json"
    trace.write_text(json.dumps(synth.trace_dict(cfg)))
    qcfg.write_text(json.dumps(synth.qconfig_dict(cfg)))
    w = gen_workload.generate_workload_from_gate_trace(str(trace), cfg.tokens, 0, str(tmp_path / "out" / "w.json"), str(qcfg))
    assert json.loads((tmp_path / "out" / "w.json").read_text()) == w
    gu, dn = w["layer-0"]["gate_up"], w["layer-0"]["down"]
    assert w["num_tokens"] == 32 and len(gu) == 65 and len(dn) == 65
    freq = json.loads(trace.read_text())["layer-0"]["access_freq"]
    for e in range(64):
        m = int(freq[e] / sum(freq) * 32 * 6)                              # gen_workload.py:88-89 floors
        assert gu[e]["shape"] == [m, 2816, 2048] and dn[e]["shape"] == [m, 2048, 1408]
    assert gu[64]["shape"] == [32, 2 * 1408 * 2, 2048] and dn[64]["shape"] == [32, 2048, 1408 * 2]
    q = json.loads(qcfg.read_text())["0"]["experts"]["64"]["gate"]
    assert dn[64]["w_bits"] == q["w_bits"]                                 # shared `down` takes the "gate" block's qcfg (:94)
    w2 = gen_workload.generate_workload_from_gate_trace(str(trace), 64, 0, None, None, "w4a4_g-1_sym")
    assert w2["layer-0"]["gate_up"][0]["a_bits"] == 4 and w2["layer-0"]["gate_up"][0]["sym"] is True
    w3 = gen_workload.generate_workload_from_gate_trace(str(trace), 64, 0, None)
    assert w3["layer-0"]["down"][3]["w_bits"] == 16


def test_template_generator_product_and_sources(tmp_path):
    tiles = {q: tile_config.get_possible_tile_list("gfx950", q)[:n] for q, n in (("w4a4_g-1_sym", 3), ("w8a8_g-1_sym", 2))}
    # w4a4 also lists the tiles on the 6-bit float path (operands as bf6 fragments); they form kernels of their own
    b6 = [t for t in tile_config.get_possible_tile_list("gfx950", "w4a4_g-1_sym") if t.is_bf6()]
    assert [t.cpp_type() for t in b6] == ["Bf6Tile<128>", "Bf6Tile<64>", "Bf6Tile<32>"] and all(t.validate() is None for t in b6)
    g = TemplateGenerator("gfx950", ["w8a8_g-1_sym", "w4a4_g-1_sym"], KernelType.Fused, tiles, out_dir=tmp_path)
    assert g.qcfgs == ["w4a4_g-1_sym", "w8a8_g-1_sym"]                     # sorted, as compose_kernel.py:82
    files = g.generate_source_code()
    assert len(g.combos) == 6 and len(files) == 7                          # 3 x 2 combinations + the ABI unit
    src = (tmp_path / "hz_fused_4.hip").read_text()
    assert 'register_fused<WxAxTile<Op::I4, 32, 256>, WxAxTile<Op::I8, 128, 256>>("groupgemm_hz_fused_4", Policy::Fused)' in src
    assert "(a_bits == 4 && w_bits == 4 && gsize == -1 && sym == true)" in src
    assert "groupgemm_hz_fused_5" in (tmp_path / "hz_fused_decl.hpp").read_text()
    # the ablation launchers are the same combinations behind another launch policy (kernel_sketch.py:148-406)
    seq = TemplateGenerator("gfx950", ["w8a8_g-1_sym", "w4a4_g-1_sym"], KernelType.Sequential, tiles, out_dir=tmp_path / "seq")
    assert len(seq.get_tile_configs()) == 6
    seq.generate_source_code()
    assert '("groupgemm_seq_launch_0", Policy::Sequential)' in (tmp_path / "seq" / "seq_launch_0.hip").read_text()
    # a tuple of tiles is a shape set: one kernel carrying every shape of the set as a branch of that format
    sets = {"w4a4_g-1_sym": [tuple(tiles["w4a4_g-1_sym"])], "w8a8_g-1_sym": [tuple(tiles["w8a8_g-1_sym"]), tiles["w8a8_g-1_sym"][0]]}
    g2 = TemplateGenerator("gfx950", ["w8a8_g-1_sym", "w4a4_g-1_sym"], KernelType.MultiStream, sets, out_dir=tmp_path / "sets")
    g2.generate_source_code()
    assert len(g2.combos) == 2
    assert ('register_fused<WxAxTile<Op::I4, 128, 256>, WxAxTile<Op::I4, 64, 256>, WxAxTile<Op::I4, 32, 256>, WxAxTile<Op::I8, 128, 256>, '
            'WxAxTile<Op::I8, 64, 256>>("groupgemm_ms_launch_0", Policy::MultiStream)') in (tmp_path / "sets" / "ms_launch_0.hip").read_text()
    with pytest.raises(ValueError, match="Unsupported qcfg"):
        TemplateGenerator("gfx950", ["w1a16_g128_sym"])
    # the reference's fp16-accumulate names are accepted and built as the base format's (fp32-accumulating) tiles
    for alias, base in (("w4a16_g128_asym_accfp16", "w4a16_g128_asym"), ("fp16_accfp16", "fp16"), ("w2a16_g-1_sym_accfp16", "w2a16_g-1_sym")):
        assert tile_config.get_info_from_qcfg_str(alias) == tile_config.get_info_from_qcfg_str(base)
        assert [t.cpp_type() for t in tile_config.get_possible_tile_list("gfx950", alias)] == [t.cpp_type() for t in tile_config.get_possible_tile_list("gfx950", base)]
    ga = TemplateGenerator("gfx950", ["w4a16_g128_asym_accfp16"], KernelType.Fused, out_dir=tmp_path / "acc")
    ga.generate_source_code()
    assert "SkinnyWoTile<4, 128" in (tmp_path / "acc" / "hz_fused_0.hip").read_text()


def test_default_library_is_generator_output(tmp_path, lib):
    """The kernels libmxmoe_amd.so registers are the generator's `default_kernel_specs`, name for name and branch for branch."""
    from mxmoe_amd.kernels import compose_kernel as ck

    specs = ck.default_kernel_specs()
    files = ck.emit_default_library(tmp_path)
    assert len(files) == len(specs) + 1                                   # one unit per kernel, and the unit that registers them in order
    src = "".join(f.read_text() for f in files)
    order = files[-1].read_text()
    assert [n for n in re.findall(r"    register_(\w+)\(\);", order)] == [name for name, _t, _c in specs]
    assert lib.mxmoe_num_kernels() == len(specs)
    policy = {ck.KernelType.Fused: 0, ck.KernelType.Sequential: 1, ck.KernelType.MultiStream: 2}
    import ctypes as C

    out = (C.c_int32 * 8)()
    for i, (name, ktype, tile_cfg) in enumerate(specs):
        assert lib.mxmoe_kernel_name(i).decode().endswith(name) and f'"{name}", {ck.POLICY[str(ktype)]}' in src
        assert lib.mxmoe_kernel_policy(i) == policy[ktype]
        tiles = ck._flat(tile_cfg.values())
        assert lib.mxmoe_kernel_num_branches(i) == len(tiles)
        for b, t in enumerate(tiles):
            assert lib.mxmoe_kernel_branch(i, b, out) == 0 and (out[1], out[2], out[3]) == (t.BM, t.BN, t.BK)


def test_run_mxmoe_gg_helpers(tmp_path):
    import run_mxmoe_gg as r

    p = tmp_path / "q-wbits5.0.json"
    p.write_text(json.dumps({**synth.qconfig_dict(synth.get_config("c5")), "LT": 1}))
    assert r.get_qcfg_list(str(p), -1) == {"w4a4_g-1_sym", "w8a8_g-1_sym", "w4a16_g128_asym"}
    assert r.get_qcfg_list(str(p), 7) == set()
    assert str(p).split("wbits")[1].split(".json")[0] == "5.0"            # workload suffix rule, run_mxmoe_gg.py:54


def test_synthetic_configs_match_the_baseline_shapes():
    c3 = synth.get_config("c3")
    ids, w = synth.make_routing(c3)
    assert ids.shape == (8192, 4) and bool((ids.sort(dim=1).values.diff(dim=1) != 0).all())   # distinct experts per token
    assert abs(float(w.sum(1).mean()) - 1) < 1e-5
    f = synth.draw_formats(c3)
    assert len(f) == 60 and {q for pair in f for q in pair} == {synth.W4A4, synth.W8A8}
    c4 = synth.get_config("c4")
    assert len(synth.draw_formats(c4)) == 65
    w13, w2 = synth.expert_weights(c4, 64)
    assert w13.shape == (2 * 2816, 2048) and w2.shape == (2048, 2816)


# ---- kernel-profile table: consumer on the reference's schema, producer pieces ----

def _ref_table():
    import json
    from pathlib import Path

    fx = json.loads((Path(__file__).parent / "golden" / "perf_table_sm89_excerpt.json").read_text())
    return fx, fx["entries"]


def test_perf_table_reference_schema():
    fx, table = _ref_table()
    assert len(fx["qcfgs"]) == 19
    assert fx["slots"]["w8a8_g-1_sym"] == ["1", "2", "3", "4"] and fx["slots"]["w4a16_g128_asym"] == ["1"]
    for q, slots in table.items():
        for s, tiles in slots.items():
            for key, rec in tiles.items():
                assert key.startswith("TileConfig(BM=") and set(rec) == {"first_iter_cost", "inc", "stderr"}


def test_perf_table_keys_round_trip_through_tile_config():
    """repr(TileConfig) is the table key: a key parsed back into a TileConfig must print as the same key."""
    from mxmoe_amd.kernels.tile_config import parse_tile_repr

    _, table = _ref_table()
    for q, slot in (("w8a8_g-1_sym", "3"), ("w4a4_g-1_sym", "3")):
        for key in table[q][slot]:
            (t,) = parse_tile_repr(key, q)
            assert repr(t) == key


def test_get_runtime_cost_known_answers():
    from mxmoe_amd.kernels.tile_config import parse_tile_repr
    from mxmoe_amd.perf_table import ProblemShape, get_runtime_cost, slot_of, table_key

    _, table = _ref_table()
    assert slot_of("w4a16_g128_asym") == "1" and slot_of("w8a8_g-1_sym") == "3"
    assert table_key("w2a16_g128_asym") == "w2a16_g128_asym_accfp16" and table_key("w4a4_g-1_sym") == "w4a4_g-1_sym"
    strategies = ["w4a4_g-1_sym", "w8a8_g-1_sym"]
    keys = {q: list(table[q]["3"])[:2] for q in strategies}
    tiles = {q: [parse_tile_repr(k, q)[0] for k in keys[q]] for q in strategies}
    work = [[ProblemShape(546, 2816, 2048), ProblemShape(546, 2048, 1408)], [ProblemShape(1, 2816, 2048), ProblemShape(1, 2048, 1408)]]
    combos, cost = get_runtime_cost(work, strategies, table, tile_cfgs=tiles)
    assert len(combos) == 4 and len(cost) == 2 and len(cost[0]) == 2 and len(cost[0][0]) == 2 and len(cost[0][0][0]) == 4
    # all four tiles are 128 x 128: ceil(546/128) * (2816/128) = 5 * 22 = 110 tiles; (2048/128) = 16 -> 80; one row -> 22 and 16
    inc = {q: [table[q]["3"][k]["inc"] for k in keys[q]] for q in strategies}
    for ci, (t4, t8) in enumerate(combos):
        i4, i8 = tiles["w4a4_g-1_sym"].index(t4), tiles["w8a8_g-1_sym"].index(t8)
        assert cost[0][0][0][ci] == inc["w4a4_g-1_sym"][i4] * 110
        assert cost[0][1][1][ci] == inc["w8a8_g-1_sym"][i8] * 80
        assert cost[1][0][1][ci] == inc["w8a8_g-1_sym"][i8] * 22
        assert cost[1][1][0][ci] == inc["w4a4_g-1_sym"][i4] * 16
    assert inc["w4a4_g-1_sym"][0] == 0.004520000000000001  # value of the reference's table itself


def test_perf_table_alias_and_weight_only_slot():
    from mxmoe_amd.perf_table import ProblemShape, get_runtime_cost

    _, table = _ref_table()

    class Tile:
        def __init__(self, key, bm, bn):
            self.key, self.BM, self.BN, self.num_warps = key, bm, bn, 4

        def __repr__(self):
            return self.key

    key = list(table["w2a16_g128_asym_accfp16"]["1"])[3]  # BM=64, BN=128
    _, cost = get_runtime_cost([[ProblemShape(100, 256, 4096)]], ["w2a16_g128_asym"], table, tile_cfgs={"w2a16_g128_asym": [Tile(key, 64, 128)]})
    assert cost == [[[[0.013920000000000002 * 4]]]]


def test_perf_table_fit_and_sweep_shapes():
    from mxmoe_amd.kernels.tile_config import get_possible_tile_list
    from mxmoe_amd.perf_table import ProblemShape, linear_fit, sweep_entry

    icpt, slope, err = linear_fit([1, 2, 3, 4], [3.0, 5.0, 7.0, 9.0])
    assert abs(icpt - 1.0) < 1e-12 and abs(slope - 2.0) < 1e-12 and err < 1e-12
    _, slope, err = linear_fit([0, 1, 2], [0.0, 1.0, 0.0])
    assert abs(slope) < 1e-12 and abs(err - (2.0 / 3 / 1 / 2) ** 0.5) < 1e-12  # rss = 2/3, n-2 = 1, sxx = 2
    for q in ("w4a4_g-1_sym", "w4a16_g128_asym"):
        for t in get_possible_tile_list("gfx950", q):
            for w in (1, 3):
                e = sweep_entry(t, q, 2048, w, cus=256)
                m, n, k = e["shape"]
                assert ProblemShape(m, n, k).num_tiles(t) == 256 * w and k == 2048


def test_build_refuses_spilling_wxax_kernels():
    """A WxAxTile kernel that spills vector registers must not be built (its hand-tracked loads would land in re-used registers)."""
    from mxmoe_amd.build import check_no_spills

    fmt = "t.hpp:1:1: remark: Function Name: {} [-Rpass-analysis=kernel-resource-usage]\nt.hpp:1:1: remark:     VGPRs Spill: {} [-Rpass-analysis=kernel-resource-usage]\n"
    check_no_spills(fmt.format("_ZN5mxmoe8WxAxTileILi1EEE", 0))
    check_no_spills(fmt.format("_ZN5mxmoe12SkinnyWoTileILi4EEE", 3))        # compiler-tracked loads: spills are only slow
    with pytest.raises(RuntimeError, match="spilled"):
        check_no_spills(fmt.format("_ZN5mxmoe8WxAxTileILi1EEE", 45))


def test_build_refuses_moves_of_registers_with_loads_in_flight():
    """The build's ISA check: a register written by a hand-tracked (inline-assembly) load may not be moved before the wait that names it."""
    from mxmoe_amd.build import check_untracked_load_copies as chk

    def kernel(body):
        return "_Z6kernelv:\n" + "\n".join(body) + "\n\ts_endpgm\n"

    load = ["\t;;#ASMSTART", "\tglobal_load_dwordx4 v[10:13], v[2:3], off", "\t;;#ASMEND"]
    wait = ["\t;;#ASMSTART", "\ts_waitcnt vmcnt(3) ; landed v[10:13]", "\t;;#ASMEND"]
    move = ["\tv_mov_b64_e32 v[20:21], v[10:11]"]
    chk(kernel(load + wait + move))                                  # copy of a landed value: fine
    chk(kernel(load + ["\tv_mov_b32_e32 v30, v31"] + wait))          # unrelated registers: fine
    with pytest.raises(RuntimeError, match="in flight"):
        chk(kernel(load + move + wait))
    with pytest.raises(RuntimeError, match="never waited"):
        chk(kernel(load))
    # whatever the mnemonic: a permute or an ordinary ALU operation reading the register, or anything overwriting it
    for bad in ("\tv_perm_b32 v40, v11, v41, v42", "\tv_and_b32_e32 v5, v10, v4", "\tv_pk_mov_b32 v[40:41], v[12:13], v[12:13]",
                "\tv_readlane_b32 s4, v13, 3", "\tv_add_u32_e32 v12, v40, v41", "\tds_write_b128 v50, v[10:13]"):
        with pytest.raises(RuntimeError, match="in flight"):
            chk(kernel(load + [bad] + wait))
        chk(kernel(load + wait + [bad]))
    chk(kernel(load + ["\tv_and_b32_e32 v5, v110, v4 ; v10 in a comment"] + wait))
    # loop: the load at the bottom of an iteration is in flight at the top of the next one
    loop = [".LBB0_1:                                ; =>This Inner Loop Header: Depth=1"] + move + wait + ["\tv_and_b32_e32 v5, v10, v4"] + load + \
           ["\ts_cbranch_scc1 .LBB0_1", ".LBB0_2:"] + wait
    with pytest.raises(RuntimeError, match="in flight"):
        chk(kernel(load + loop))
    ok_loop = [".LBB0_1:                                ; =>This Inner Loop Header: Depth=1"] + wait + move + load + ["\ts_cbranch_scc1 .LBB0_1", ".LBB0_2:"] + wait
    chk(kernel(load + ok_loop))


def test_build_refuses_compiler_memory_instructions_in_hand_counted_loops():
    from mxmoe_amd.build import check_untracked_load_copies as chk

    load = ["\t;;#ASMSTART", "\tglobal_load_dwordx4 v[10:13], v[2:3], off", "\t;;#ASMEND"]
    wait = ["\t;;#ASMSTART", "\ts_waitcnt vmcnt(3) ; landed v[10:13]", "\t;;#ASMEND"]
    head = [".LBB0_1:                                ; =>This Inner Loop Header: Depth=1"]
    tail = ["\ts_cbranch_scc1 .LBB0_1", ".LBB0_2:"]
    mk = lambda body: "_Z6kernelv:\n" + "\n".join(load + head + body + tail + wait) + "\n\ts_endpgm\n"
    chk(mk(wait + load))
    with pytest.raises(RuntimeError, match="counted by hand"):
        chk(mk(wait + load + ["\tglobal_load_dword v40, v[2:3], off"]))     # in flight around the back edge
    chk(mk(wait + ["\tglobal_load_dword v40, v[2:3], off"] + load))         # between the wait and the next load nothing is in flight
    # kernels without hand-tracked loads may hold any memory instruction
    chk("_Z6kernelv:\n" + "\n".join(head + ["\tglobal_load_dword v40, v[2:3], off"] + tail) + "\n\ts_endpgm\n")
    # outside loops as well: between the first hand-counted load and the last hand-placed wait nothing may be added ...
    dma = ["\t;;#ASMSTART", "\ts_mov_b32 m0, s4", "\tbuffer_load_dwordx4 v1, s[8:11], s5 offen lds", "\t;;#ASMEND"]
    plain_wait = ["\t;;#ASMSTART", "\ts_waitcnt vmcnt(0)", "\t;;#ASMEND"]
    straight = lambda body: "_Z6kernelv:\n" + "\n".join(body) + "\n\ts_endpgm\n"
    for extra in ("\tglobal_load_dword v40, v[2:3], off", "\tglobal_store_dword v[2:3], v40, off", "\tbuffer_load_dword v40, v41, s[8:11], 0 offen",
                  "\tscratch_store_dword off, v40, s32"):
        with pytest.raises(RuntimeError, match="counted by hand"):
            chk(straight(load + [extra] + wait))
        # direct-to-LDS loads land in no register: compiler loads behind them only lengthen the hand-placed wait (loads retire in
        # order), but writes retire out of order with loads and would make the count meaningless
        if "_load" in extra and not extra.strip().startswith("scratch"):
            chk(straight(dma + [extra] + plain_wait))
        else:
            with pytest.raises(RuntimeError, match="counted by hand"):
                chk(straight(dma + [extra] + plain_wait))
        # before the first and after the last of them the compiler is free
        chk(straight([extra] + load + wait + [extra]))
        chk(straight([extra] + dma + plain_wait + [extra]))
    # the state follows the branches, not the layout: a block laid out after the wait but entered from before it is judged in flight
    cold = "_Z6kernelv:\n" + "\n".join(load + ["\ts_cbranch_scc1 .LBB0_9", ".LBB0_1:"] + wait + ["\ts_endpgm", ".LBB0_9:",
                                                "\tv_mov_b32_e32 v40, v11", "\ts_branch .LBB0_1"]) + "\n"
    with pytest.raises(RuntimeError, match="in flight"):
        chk(cold)
    # ... and a block laid out in the middle of the loads but only reached after the wait is not
    chk("_Z6kernelv:\n" + "\n".join(["\ts_branch .LBB0_2", ".LBB0_1:", "\tv_mov_b32_e32 v40, v11", "\ts_endpgm", ".LBB0_2:"] + load + wait +
                                    ["\ts_branch .LBB0_1"]) + "\n")
    # a hand-placed wait for vmcnt(0) lands everything
    chk(straight(load + plain_wait + ["\tv_mov_b32_e32 v40, v11"]))


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits non-zero without touching a device."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    res = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and "one GPU" in res.stderr and res.stdout.strip() == ""


def test_harness_input_parsers(tmp_path):
    """test.cu:611-691: workload JSON files (every key but "num_tokens" is a case) and the legacy text form
    `a_bits-w_bits-gsize-sym MxNxK`, one problem per line."""
    from mxmoe_amd import harness

    cfg = synth.get_config("c4")
    trace, qcfg = tmp_path / "moe-gate.json", tmp_path / "q-wbits4.json"
    trace.write_text(json.dumps(synth.trace_dict(cfg)))
    qcfg.write_text(json.dumps(synth.qconfig_dict(cfg)))
    w = tmp_path / "w.json"
    gen_workload.generate_workload_from_gate_trace(str(trace), cfg.tokens, 0, str(w), str(qcfg))
    cases = harness.parse_input_file(str(w))
    assert list(cases) == ["layer-0"] and len(cases["layer-0"]["gate_up"]) == 65 and set(cases["layer-0"]["down"][0]) >= {"shape", "w_bits", "a_bits", "gsize", "sym"}
    legacy = tmp_path / "cases.txt"
    legacy.write_text("4-4--1-sym 512x2816x2048\n16-4-128-asym 32x2048x1408\n\n8x8x-1xsym 7,256,128\n")
    got = harness.parse_input_file(str(legacy))
    assert list(got) == ["test_case"] and list(got["test_case"]) == ["gate_up"]
    assert got["test_case"]["gate_up"] == [
        {"shape": [512, 2816, 2048], "w_bits": 4, "a_bits": 4, "gsize": -1, "sym": True},
        {"shape": [32, 2048, 1408], "w_bits": 4, "a_bits": 16, "gsize": 128, "sym": False},
        {"shape": [7, 256, 128], "w_bits": 8, "a_bits": 8, "gsize": -1, "sym": True}]
    legacy.write_text("4-3-128-asym 1x256x128\n")
    with pytest.raises(ValueError, match="Ava w bits"):                      # test.cu:633-636 lists 16 / 8 / 4 / 2
        harness.parse_input_file(str(legacy))
    with pytest.raises(FileNotFoundError):
        harness.parse_input_file(str(tmp_path / "none.json"))


def test_run_mxmoe_gg_up_to_the_library(tmp_path, monkeypatch):
    """The CLI end to end without a GPU: synthetic trace and qconfig -> qcfg set -> workload JSON -> generated sources -> hipcc
    -> a library that loads and registers the generated kernel (run_mxmoe_gg.py:34-111 up to the bench subprocess)."""
    import run_mxmoe_gg as r
    from mxmoe_amd import _lib
    from mxmoe_amd.kernels import compose_kernel as ck

    monkeypatch.setattr(r, "CUR_DIR", str(tmp_path))
    monkeypatch.setattr(ck, "GEN_DIR", tmp_path / "generated")
    assert r.main(["--synthetic", "c4", "--max-kernels", "1", "--no-bench"]) == 0
    wl = json.loads((tmp_path / "out" / "workloads" / "ds2-synthetic-32--c4.json").read_text())
    assert wl["num_tokens"] == 32 and len(wl["layer-0"]["gate_up"]) == 65
    assert {(e["w_bits"], e["a_bits"], e["gsize"]) for e in wl["layer-0"]["down"]} == {(4, 16, 128), (3, 16, 128)}
    libs = list((tmp_path / "generated").glob("libmxmoe_hz_fused_*.so"))
    assert len(libs) == 1
    lib = _lib.load(libs[0])
    assert lib.mxmoe_num_kernels() == 1
    name = lib.mxmoe_kernel_name(0).decode()
    assert name.endswith("groupgemm_hz_fused_0") and "w4a16_g128_asym" in name and "w3a16_g128_asym" in name
