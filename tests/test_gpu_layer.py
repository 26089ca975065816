"""Whole-layer GPU parity: permute -> (Hadamard) quantise -> gate_up GroupGEMM -> SiLU*up -> (Hadamard) quantise -> down GroupGEMM,
every intermediate integer accumulator compared bit for bit with the CPU oracle chain on the same seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
F16 = np.float16


def _rel(a, b):
    a, b = a.astype(np.float64), b.astype(np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-6)


def _oracle_block(x, w, qp, rotate_mode):
    tag = O.act_tag(qp[0], qp[2])
    rot = rotate_mode == 2 or (rotate_mode == 1 and tag != 0)
    return O.linear_block(x, w, qp, rot) if qp[0] < 16 else O.linear_block(O.online_hadamard(x) if rot else x, w, qp, False)


def _run(cfg, formats, bf6=False):
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    hidden = synth.make_hidden(cfg)
    ids, _ = synth.make_routing(cfg)
    weights = [synth.expert_weights(cfg, e) for e in range(cfg.num_experts + (1 if cfg.num_shared else 0))]
    layer = MxMoELayer(cfg, formats=formats, weights=weights, bf6=bf6)
    outs = layer.forward(hidden, ids, dump_acc=True)
    torch.cuda.synchronize()
    st = layer.state
    _, perm, _, recv = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    assert np.array_equal(st["recv"].numpy(), recv)
    h = hidden.numpy()
    p = row = 0
    results = []
    for e in range(len(weights)):
        m = cfg.tokens if e == cfg.num_experts else int(recv[e])
        if m == 0:
            continue
        x = h if e == cfg.num_experts else h[perm[row:row + m]]
        if e < cfg.num_experts:
            row += m
        w13, w2 = weights[e][0].numpy(), weights[e][1].numpy()
        mid_k, mid_f, acc1 = _oracle_block(x, w13, formats[e][0], cfg.rotate)
        y = O.silu_mul(mid_k)
        out_k, out_f, acc2 = _oracle_block(y, w2, formats[e][1], cfg.rotate)
        results.append(dict(e=e, acc1=acc1, acc2=acc2, mid=mid_k, out=out_k, out_f=out_f,
                            g_acc1=st["acc1"][p].cpu().numpy(), g_acc2=st["acc2"][p].cpu().numpy(),
                            g_mid=st["mid"][p].cpu().numpy(), g_out=outs[p].cpu().numpy()))
        p += 1
    assert p == len(outs)
    return results


@pytest.mark.parametrize("bf6", [False, True])
def test_wxax_layer_is_bit_exact_end_to_end(bf6):
    """bf6: the w4a4 blocks on the 6-bit float matrix path (weights and activations as bf6 fragments): the same bits."""
    from mxmoe_amd import synth

    cfg = synth.MoEConfig("t", "test", 5, 2, 256, 1408, 40 if not bf6 else 150, num_shared=0, rotate=1)
    fm = [(synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4), (synth.W4A4, synth.W4A4), (synth.W8A8, synth.W8A8), (synth.W4A4, synth.W8A8)]
    for r in _run(cfg, fm, bf6):
        assert np.array_equal(r["g_acc1"], r["acc1"]), f"gate_up accumulators, expert {r['e']}"
        assert np.array_equal(r["g_mid"].view(np.uint16), r["mid"].view(np.uint16)), f"gate_up fp16, expert {r['e']}"
        assert np.array_equal(r["g_acc2"], r["acc2"]), f"down accumulators, expert {r['e']}"
        assert np.array_equal(r["g_out"].view(np.uint16), r["out"].view(np.uint16)), f"down fp16, expert {r['e']}"
        assert _rel(r["g_out"], r["out_f"]) <= 1e-2                         # vs the fake-quant path


def test_layer_with_group_quantised_experts_is_bit_exact():
    """Experts in w4a4_g128_sym next to per-channel ones: quantiser (one scale per 128 values), both GroupGEMMs and the fp16 results
    equal the oracle's bit for bit (the accumulators of the group format are fp32 sums and are compared in the GroupGEMM's own test)."""
    from mxmoe_amd import synth

    cfg = synth.MoEConfig("t", "test", 4, 2, 256, 1408, 40, num_shared=0, rotate=1)
    g = synth.W4A4G128
    fm = [(g, g), (synth.W8A8, g), (g, synth.W4A4), (synth.W4A4, synth.W8A8)]
    for r in _run(cfg, fm):
        assert np.array_equal(r["g_mid"].view(np.uint16), r["mid"].view(np.uint16)), f"gate_up fp16, expert {r['e']}"
        assert np.array_equal(r["g_out"].view(np.uint16), r["out"].view(np.uint16)), f"down fp16, expert {r['e']}"
        assert _rel(r["g_out"], r["out_f"]) <= 1e-2


def test_mixed_layer_with_shared_expert_within_tolerance():
    from mxmoe_amd import synth

    cfg = synth.MoEConfig("t", "test", 4, 2, 256, 1408, 16, num_shared=2, rotate=0)
    w8a16, w4a16_pc = (16, 8, 128, False), (16, 4, -1, True)   # 8-bit weights; 4-bit weights with one scale per channel
    fm = [(synth.W4A16, synth.W3A16), (w8a16, synth.W4A16), (synth.FP16, w8a16), (w4a16_pc, synth.W4A16), (synth.W4A16, synth.W3A16)]
    for r in _run(cfg, fm):
        assert _rel(r["g_mid"], r["mid"]) <= 1e-2, f"gate_up, expert {r['e']}"
        # the down input differs in the last fp16 bit from the oracle's, so compare the end result at the stated tolerance
        assert _rel(r["g_out"], r["out"]) <= 1e-2, f"down, expert {r['e']}"


def test_unpermute_combine_bit_exact():
    """The step after the down launch against the oracle: routed only, with a shared expert, and with dropped expert ids."""
    from mxmoe_amd import ops

    rng = np.random.default_rng(11)
    for (t, k, e, n, shared, drop) in [(50, 4, 8, 256, False, False), (33, 6, 16, 1408, True, False), (17, 2, 4, 2048, True, True), (1, 1, 1, 8, False, False)]:
        ids = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
        if drop:
            ids[::3, 0] = e + 5                  # ids outside [0, E) are dropped by the permutation
        _, _, slot, recv = O.permute_by_expert(np.where(ids < e, ids, e), e + 1)
        rows_n = int(recv[:e].sum())
        slot = slot[:rows_n]
        rows = rng.standard_normal((rows_n, n)).astype(F16)
        sh = rng.standard_normal((t, n)).astype(F16) if shared else None
        w = rng.random((t, k)).astype(np.float32)
        store = np.concatenate([rows.reshape(-1)] + ([sh.reshape(-1)] if shared else []))
        out = ops.gg_unpermute_out(torch.from_numpy(store).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(w).cuda(), e, n, 2 if shared else 0)
        ref = O.unpermute_combine(rows, slot, w, sh)
        assert np.array_equal(out.cpu().numpy().view(np.uint16), ref.view(np.uint16)), (t, k, e, n, shared, drop)


def test_layer_combine_end_to_end():
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 6, 2, 256, 1408, 48, num_shared=2, rotate=1, formats=(synth.W4A4, synth.W8A8), format_probs=(0.5, 0.5))
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    layer = MxMoELayer(cfg)
    outs = layer.forward(hidden, ids)
    final = layer.combine(w)
    torch.cuda.synchronize()
    assert torch.equal(layer(hidden, ids, w), final)              # the one-call form
    outs = layer.state["out"]
    _, _, slot, recv = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    rows = np.concatenate([o.cpu().numpy() for o in outs[:-1]])
    ref = O.unpermute_combine(rows, slot, w.numpy(), outs[-1].cpu().numpy())
    assert final.shape == (cfg.tokens, cfg.hidden)
    assert np.array_equal(final.cpu().numpy().view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("num_shared,rotate,drop", [(0, 1, False), (2, 1, False), (1, 0, True), (0, 2, True)])
def test_one_call_form_equals_the_stepwise_forward(num_shared, rotate, drop):
    """`layer(hidden, ids, weights)` builds all host tables in one pass; it must give exactly the result of the operator-by-operator
    path for every format family, with a shared expert, with experts that receive no row and with expert ids out of range (dropped)."""
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 8, 2, 256, 1408, 40, num_shared=num_shared, rotate=rotate)
    g = synth.W4A4G128
    fm = [(synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4), (g, g), (synth.W4A16, synth.W3A16), (synth.FP16, synth.FP16), (synth.W4A4, synth.W4A4),
          (synth.W8A8, g), (synth.W3A16, synth.W4A16)]
    if num_shared:
        fm.append((synth.W4A16, synth.W4A16) if rotate == 0 else (synth.W8A8, synth.W4A4))
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids = torch.where(ids == 5, torch.full_like(ids, 1), ids)      # expert 5 receives nothing
    if drop:
        ids = torch.where(ids == 3, torch.full_like(ids, cfg.num_experts), ids)   # as on a GPU that does not own expert 3
    layer = MxMoELayer(cfg, formats=fm)
    layer.forward(hidden, ids)
    stepwise = layer.combine(w).clone()
    one_call = layer(hidden, ids, w)
    torch.cuda.synchronize()
    assert int(layer.state["recv"][5]) == 0
    assert torch.equal(one_call, stepwise)
    assert torch.equal(layer(hidden, ids, w), stepwise)            # and again: nothing is left over from the previous call


def test_layer_from_checkpoint_file_keeps_the_function(tmp_path):
    """fp16 weights -> rotate + quantise + pack -> file -> layer: identical to packing in place, and (the weight rotation cancelling
    the online rotation of the activations) still the function of the fp16 MLP up to w8a8 quantisation noise."""
    from mxmoe_amd import checkpoint as C
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "qwen2_moe", 4, 2, 256, 1408, 64, rotate=1, formats=(synth.W8A8,), format_probs=(1.0,))
    formats = [(synth.W8A8, synth.W8A8)] * cfg.num_experts
    experts = [synth.expert_weights(cfg, e) for e in range(cfg.num_experts)]
    tensors, meta = C.pack_layer(experts, formats, rotate=1, model="qwen2_moe")
    path = str(tmp_path / "layer.safetensors")
    C.save_layer(path, tensors, meta)
    w13, w2, _ = C.load_layer(path, device="cuda")
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)

    from_file = MxMoELayer(cfg, packed=(w13, w2))
    from_file.forward(hidden, ids)
    a = from_file.combine(w).cpu()
    in_place = MxMoELayer(cfg, formats=formats, weights=[(C.rotate_input_weights(w13_), C.rotate_input_weights(w2_)) for w13_, w2_ in experts])
    in_place.forward(hidden, ids)
    b = in_place.combine(w).cpu()
    assert torch.equal(a, b)

    # the fp16 MLP with the ORIGINAL weights, fp32 arithmetic
    x = hidden.float()
    ref = torch.zeros(cfg.tokens, cfg.hidden)
    for t in range(cfg.tokens):
        for j in range(cfg.topk):
            w13_, w2_ = experts[int(ids[t, j])]
            h = w13_.float() @ x[t]
            g, u = h[:cfg.inter], h[cfg.inter:]
            ref[t] += float(w[t, j]) * (w2_.float() @ (g * torch.sigmoid(g) * u))
    assert _rel(a.float().numpy(), ref.numpy()) <= 5e-2


def test_layer_from_fake_quantised_weights_is_their_function(tmp_path):
    """Weights already on a quantisation grid (what a GPTQ run saves) are packed with their own codes: with fp16 activations
    (w4a16 / w3a16 blocks) the layer is the MLP of exactly those weights, to fp16 rounding; re-quantising them by min / max would
    add a second quantisation error."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from test_checkpoint import _gptq_like
    from mxmoe_amd import checkpoint as C
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "qwen2_moe", 4, 2, 256, 384, 48, rotate=0, formats=(synth.W4A16,), format_probs=(1.0,))
    formats = [(synth.W4A16, synth.W3A16)] * cfg.num_experts
    experts = []
    for e in range(cfg.num_experts):
        w13, _, _ = _gptq_like(2 * cfg.inter, cfg.hidden, 4, 128, False, torch.bfloat16, 100 + e)
        w2, _, _ = _gptq_like(cfg.hidden, cfg.inter, 3, 128, False, torch.bfloat16, 200 + e)
        experts.append((w13, w2))
    tensors, meta = C.pack_layer(experts, formats, rotate=0, model="qwen2_moe", fake_quant=True)
    path = str(tmp_path / "gptq_layer.safetensors")
    C.save_layer(path, tensors, meta)
    w13p, w2p, _ = C.load_layer(path, device="cuda")
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    layer = MxMoELayer(cfg, packed=(w13p, w2p))
    out = layer(hidden, ids, w).float().cpu()

    def mlp(ws):
        x = hidden.float().cpu()
        ref = torch.zeros(cfg.tokens, cfg.hidden)
        for t in range(cfg.tokens):
            for j in range(cfg.topk):
                w13_, w2_ = ws[int(ids[t, j])]
                h = (w13_.float() @ x[t]).half().float()
                g, u = h[:cfg.inter], h[cfg.inter:]
                ref[t] += float(w[t, j]) * (w2_.float() @ (g * torch.sigmoid(g) * u).half().float())
        return ref

    ref = mlp(experts)
    err = _rel(out.numpy(), ref.numpy())
    assert err <= 4e-3, err
    # the same weights quantised a second time by min / max are measurably further from their own function
    requant = MxMoELayer(cfg, formats=formats, weights=[(a.half(), b.half()) for a, b in experts])
    err2 = _rel(requant(hidden, ids, w).float().cpu().numpy(), ref.numpy())
    assert err2 > 3 * err, (err, err2)


def _small_layer(num_shared=1, rotate=1, bf6=False, hidden=256, topk=2):
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 6, topk, hidden, 1408, 96, num_shared=num_shared, rotate=rotate)
    g = synth.W4A4G128
    fm = [(synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4), (g, g), (synth.W4A16, synth.W3A16), (synth.FP16, synth.FP16), (synth.W4A4, synth.W4A4),
          (synth.W8A8, synth.W8A8)][: 6 + (1 if num_shared else 0)]
    return cfg, MxMoELayer(cfg, formats=fm, bf6=bf6)


@pytest.mark.parametrize("num_shared", [0, 1])
def test_planned_forward_equals_the_host_planned_one(num_shared):
    """The forward whose tables a device kernel derives from the counts (no synchronisation) against the forward whose tables the
    host builds after reading the counts back, and against the stepwise operators: identical bits, every format in one layer; the
    device-built tables themselves equal the host's."""
    from mxmoe_amd import _lib, synth
    from mxmoe_amd import layer_tables as LT

    cfg, layer = _small_layer(num_shared)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids[5:9, 0] = 2                                                     # one expert much busier than the others
    layer.forward(hidden, ids)
    want = layer.combine(w).clone()
    got = layer(hidden, ids, w)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert torch.equal(layer.call_with_host_tables(hidden, ids, w), want)
    # the planner's tables: quantiser table, pointers and sizes of the first launch against the array-arithmetic version
    lib = _lib.load()
    ps = layer._planned_setup(cfg.tokens, cfg.topk)
    et = layer.n_exp_total
    raw = ps["b1"]["plan"].cpu().numpy()
    off = [lib.mxmoe_plan_offset(i, et) for i in range(6)]
    table = raw[off[1]:off[1] + 32 * et].view(np.int64).reshape(4, et)
    ptrs = raw[off[2]:off[2] + 40 * et].view(np.int64).reshape(5, et)
    misc = raw[off[3]:off[3] + 16].view(np.int64)
    sizes = raw[off[4]:off[4] + 12 * et].view(np.uint32).reshape(et, 3)
    gu, _dn = layer._static_tables()
    rows = np.concatenate([np.bincount(ids.numpy().reshape(-1), minlength=cfg.num_experts), [cfg.tokens] * (1 if num_shared else 0)]).astype(np.int64)
    bt = LT.block_tables(gu, rows)
    assert np.array_equal(table, bt.table)
    assert misc[0] == rows[: cfg.num_experts].sum()
    assert np.array_equal(sizes, np.stack([rows, gu.n, gu.k], axis=1).astype(np.uint32))
    b1 = ps["b1"]
    assert np.array_equal(ptrs[0], b1["inp"].data_ptr() + 2 * bt.table[2]) and np.array_equal(ptrs[4], ps["mid"].data_ptr() + 2 * bt.out_off)
    assert np.array_equal(ptrs[1], gu.b_ptr) and np.array_equal(ptrs[3], gu.sb_ptr)
    assert np.array_equal(ptrs[2], np.where(gu.sld > 0, b1["scale"].data_ptr() + 2 * bt.table[3], 0))
    assert misc[1] == (ptrs[4][-1] if num_shared else 0)


@pytest.mark.parametrize("hidden,topk,rotate", [(512, 2, 1), (1024, 5, 2), (512, 3, 0)])
def test_planned_forward_with_the_per_token_prologue_equals_the_per_row_one(hidden, topk, rotate):
    """Power-of-two rows: the planned forward quantises its input once per token and format (mxmoe_quant_act_tokens), the forward
    with host tables once per destination row (mxmoe_quant_act); every format in one layer, a shared expert, some expert ids out
    of range.  Identical outputs."""
    from mxmoe_amd import synth

    cfg, layer = _small_layer(1, rotate, hidden=hidden, topk=topk)
    hidden_t = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids[3, 0] = cfg.num_experts + 1
    ids[7, topk - 1] = -2
    assert layer._planned_setup(cfg.tokens, cfg.topk)["per_token"]
    got = layer(hidden_t, ids, w).clone()
    want = layer.call_with_host_tables(hidden_t, ids, w)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_device_planner_writes_the_host_launchers_tile_tables():
    """Entries, phases and totals that the planning kernel writes against the host launcher's for the same counts, on a layer whose
    shared expert is twice as wide as the routed ones (its tiles run first inside their branch) and with experts left empty."""
    import ctypes as C

    from mxmoe_amd import _lib, synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 9, 2, 256, 1408, 70, num_shared=2, formats=(synth.W4A16, synth.W3A16, synth.W4A4, synth.W8A8), format_probs=(0.3, 0.2, 0.3, 0.2))
    layer = MxMoELayer(cfg)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids = torch.where(ids == 4, torch.full_like(ids, 6), ids)            # expert 4 receives nothing
    layer.forward(hidden, ids)
    want = layer.combine(w).clone()
    assert torch.equal(layer(hidden, ids, w), want)
    lib = _lib.load()
    ps = layer._planned_setup(cfg.tokens, cfg.topk)
    et = layer.n_exp_total
    rows = np.concatenate([np.bincount(ids.numpy().reshape(-1), minlength=cfg.num_experts), [cfg.tokens]])
    for blk, qps in (("b1", layer.qp_gate_up), ("b2", layer.qp_down)):
        b = ps[blk]
        h_sizes = (_lib.Dim3 * et)(*[_lib.Dim3(int(rows[e]), b["h"][e].N, b["h"][e].K) for e in range(et)])
        h_q = (_lib.QParams * et)(*[_lib.QParams(int(q[0]), int(q[1]), int(q[2]), 1 if q[3] else 0) for q in qps])
        out = (C.c_int32 * 1200)()
        assert lib.mxmoe_group_gemm_plan_tables(b["kid"], h_sizes, h_q, et, out, 1200) == 0, lib.mxmoe_last_error()
        host = np.array(out[:], dtype=np.int32)
        ne, tiles, nph, grid = host[:4]
        hdr = b["plan"].cpu().numpy()[:4096].view(np.int32)
        base = 56 // 4                                                  # seven pointers, then the integers of the table
        assert (hdr[base], hdr[base + 1], hdr[base + 2], hdr[base + 3]) == (0, ne, tiles, nph)
        assert np.array_equal(hdr[base + 4: base + 4 + nph + 1], host[4: 4 + nph + 1])                  # phase_tile0
        assert np.array_equal(hdr[base + 13: base + 13 + nph + 1], host[13: 13 + nph + 1])              # phase_wg0
        assert np.array_equal(hdr[base + 23: base + 23 + 4 * ne], host[22: 22 + 4 * ne])                # entries, in launch order (after phase_flat)
        assert grid <= b["grid"]
        if blk == "b2":                                                 # the shared expert's down block is the long one: first of its branch
            first_problems = [int(host[22 + 4 * i + 3]) & 0xFFFF for i in range(ne)]
            br = [int(host[22 + 4 * i + 3]) >> 16 for i in range(ne)]
            sh_at = first_problems.index(cfg.num_experts)
            assert sh_at == br.index(br[sh_at])


def test_planned_forward_drops_out_of_range_experts_like_the_operators():
    from mxmoe_amd import synth

    cfg, layer = _small_layer(1)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids[::7, 1] = cfg.num_experts + 2                                   # these slots belong to experts this GPU does not hold
    layer.forward(hidden, ids)
    want = layer.combine(w).clone()
    got = layer(hidden, ids, w)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and bool(torch.isfinite(got).all())


def test_planned_forward_without_any_tile_after_a_forward_with_tiles():
    """Every routed id belongs to experts this GPU does not hold and there is no shared expert: both launches have no tile.  The
    plan buffers still hold the previous forward's tables (they are reused between calls), and the launches run with their
    worst-case grids; the result is all zeros, as the host-planned forward gives."""
    from mxmoe_amd import synth

    cfg, layer = _small_layer(0)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    first = layer(hidden, ids, w).clone()                               # fills the plan buffers with a real plan
    torch.cuda.synchronize()
    assert bool((first != 0).any())
    away = torch.full_like(ids, cfg.num_experts + 1)
    got = layer(hidden, away, w)
    torch.cuda.synchronize()
    assert torch.equal(got, torch.zeros_like(got))
    assert torch.equal(layer.call_with_host_tables(hidden, away, w), got)
    assert torch.equal(layer(hidden, ids, w), first)                    # and the buffers serve the next real forward


@pytest.mark.parametrize("num_shared", [0, 1])
def test_layer_on_the_bf6_matrix_path_gives_the_same_bits_in_every_form(num_shared):
    """A layer whose w4a4 blocks run on the 6-bit float matrix path (every format in one layer, so the mixed kernel): stepwise
    operators, host-planned forward, device-planned forward and the layer without bf6 all return identical outputs."""
    from mxmoe_amd import synth

    cfg, plain = _small_layer(num_shared)
    _, layer = _small_layer(num_shared, bf6=True)
    assert layer.kid_gate_up >= 0 and layer.kid_down >= 0 and plain.kid_gate_up == -1
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids[5:40, 0] = 5                                                    # a w4a4 expert with more than one block of rows
    plain.forward(hidden, ids)
    want = plain.combine(w).clone()
    layer.forward(hidden, ids)
    assert torch.equal(layer.combine(w), want)
    assert torch.equal(layer.call_with_host_tables(hidden, ids, w), want)
    assert torch.equal(layer(hidden, ids, w), want)
    ids2 = torch.where(ids == 0, torch.full_like(ids, 1), ids)          # another routing through the same buffers
    plain.forward(hidden, ids2)
    assert torch.equal(layer(hidden, ids2, w), plain.combine(w))


def test_layer_with_w8a8_blocks_in_fp8():
    """MxMoELayer(fp8=True): the w8a8 blocks of a mixed w4a4 / w8a8 layer in e4m3 (weights, activations, fp8 matrix instruction).
    Stepwise operators, host-planned and device-planned forwards agree bit for bit with each other (same kernels, same order of
    additions), and each block of every expert is within 1e-3 of the oracle's block in that format on the same input."""
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 4, 2, 256, 1408, 60, num_shared=0, rotate=1)
    fm = [(synth.W8A8, synth.W8A8), (synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4), (synth.W4A4, synth.W4A4)]
    weights = [synth.expert_weights(cfg, e) for e in range(4)]
    layer = MxMoELayer(cfg, formats=fm, weights=weights, fp8=True)
    assert layer.kid_gate_up >= 0
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    outs = [o.cpu().numpy() for o in layer.forward(hidden, ids)]
    want = layer.combine(w).clone()
    assert torch.equal(layer(hidden, ids, w), want) and torch.equal(layer.call_with_host_tables(hidden, ids, w), want)
    _, perm, _, recv = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    row = p = 0
    for e in range(4):
        m = int(recv[e])
        if m == 0:
            continue
        x = hidden.numpy()[perm[row:row + m]]
        row += m

        def block(inp, wt, qp):
            return O.linear_block_fp8(inp, wt, True)[0] if qp == synth.W8A8 else O.linear_block(inp, wt, qp, True)[0]

        # block by block, the second one on the intermediate the GPU produced: a last-bit difference in the first block's fp32 sums can
        # move an e4m3 code of the second block's input by a whole step of that coarse format, which is no error of either block
        mid = block(x, weights[e][0].numpy(), fm[e][0])
        g_mid = layer.state["mid"][p].cpu().numpy()
        assert _rel(g_mid, mid) <= 1e-3, (e, _rel(g_mid, mid))
        ref = block(O.silu_mul(g_mid), weights[e][1].numpy(), fm[e][1])
        assert np.isfinite(outs[p]).all() and _rel(outs[p], ref) <= 1e-3, (e, _rel(outs[p], ref))
        p += 1


def test_fp8_blocks_next_to_every_other_format():
    """fp8=True in a layer that also holds fp16, weight-only and group-quantised blocks (kernel groupgemm_hz_fused_all_e4m3): the three
    forms of the forward agree bit for bit, and the result is within 1e-1 (of the largest output) of the same layer with int8 w8a8
    blocks: e4m3 keeps 3 mantissa bits where int8 keeps up to 7, so the two formats of the same block differ by a few per cent."""
    from mxmoe_amd import _lib, synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 6, 3, 512, 1408, 70, num_shared=1, rotate=1)
    fm = [(synth.W8A8, synth.W4A16), (synth.FP16, synth.W8A8), (synth.W4A4G128, synth.W8A8), ((16, 8, 128, False), synth.W4A4), (synth.W8A8, synth.W8A8),
          (synth.W3A16, synth.W2A16), (synth.W8A8, synth.W8A8)]
    weights = [synth.expert_weights(cfg, e) for e in range(7)]
    layer = MxMoELayer(cfg, formats=fm, weights=weights, fp8=True)
    lib = _lib.load()
    assert lib.mxmoe_kernel_name(layer.kid_gate_up).decode().endswith("groupgemm_hz_fused_all_e4m3")
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    layer.forward(hidden, ids)
    want = layer.combine(w).clone()
    assert torch.equal(layer(hidden, ids, w), want) and torch.equal(layer.call_with_host_tables(hidden, ids, w), want)
    ref = MxMoELayer(cfg, formats=fm, weights=weights)(hidden, ids, w)
    assert _rel(want.float().cpu().numpy(), ref.float().cpu().numpy()) <= 1e-1


def test_planned_forward_of_more_experts_than_one_launch_holds():
    """130 routed experts and a shared one: each block runs as two launches (experts 0 .. 119, then the rest), planned on the device
    chunk by chunk; the result equals the stepwise operators' (whose host launcher splits long problem lists the same way) and the
    host-planned forward's, also with experts left empty and with dropped ids."""
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 130, 3, 256, 512, 120, num_shared=1, rotate=1, formats=(synth.W4A4, synth.W8A8, synth.FP16), format_probs=(0.4, 0.4, 0.2))
    layer = MxMoELayer(cfg)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids = torch.where(ids == 125, torch.full_like(ids, 7), ids)         # an expert of the second launch receives nothing
    for trial in range(2):
        layer.forward(hidden, ids)
        want = layer.combine(w).clone()
        got = layer(hidden, ids, w)
        torch.cuda.synchronize()
        assert torch.equal(got, want), trial
        assert torch.equal(layer.call_with_host_tables(hidden, ids, w), want)
        ids = ids.clone()
        ids[::5, 1] = cfg.num_experts + 3                                # second round: some slots belong to experts held elsewhere


@pytest.mark.parametrize("experts,tokens", [(6, 700), (130, 500)])
def test_two_launch_permutation_and_planning_writes_what_the_separate_calls_write(experts, tokens):
    """mxmoe_permute_plan_layer_ws (count; scatter + plan side by side) against mxmoe_build_permutation_inv + mxmoe_plan_layer (four
    launches) on the same buffers: identical permutation, counts, inverse map and plan buffers, with dropped ids; the forward that
    uses it equals the stepwise operators' result."""
    import ctypes as C

    from mxmoe_amd import _lib, synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", experts, 3, 256, 512, tokens, num_shared=1, rotate=1, formats=(synth.W4A4, synth.W8A8, synth.FP16), format_probs=(0.4, 0.4, 0.2))
    layer = MxMoELayer(cfg)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids = ids.clone()
    ids[::7, 2] = experts + 1                                            # dropped slots
    ids[3, 0] = -1
    layer.forward(hidden, ids)
    want = layer.combine(w).clone()
    got = layer(hidden, ids, w)                                          # (more than 256 entries: the two-launch head)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    lib = _lib.load()
    ps = layer._planned_setup(tokens, cfg.topk)
    assert ps["r_cap"] > 256 and -(-ps["r_cap"] // 256) * experts <= 16384
    names = ("dst", "perm", "slot", "recv", "row_of_slot")
    routed = int(((ids >= 0) & (ids < experts)).sum())
    snap = {k: ps[k].clone() for k in names}
    plans = [ps["b1"]["plan"].clone(), ps["b2"]["plan"].clone()]
    for k in names:
        ps[k].fill_(-3)
    ps["b1"]["plan"].zero_()
    ps["b2"]["plan"].zero_()
    stream = torch.cuda.current_stream().cuda_stream
    d_ids = ids.to("cuda").to(torch.int32).contiguous()
    _lib.check(lib, lib.mxmoe_build_permutation_inv(d_ids.data_ptr(), tokens, cfg.topk, experts, ps["dst"].data_ptr(), ps["perm"].data_ptr(), ps["slot"].data_ptr(),
                                                    ps["recv"].data_ptr(), ps["row_of_slot"].data_ptr(), ps["perm_ws"].data_ptr(), stream))
    _lib.check(lib, lib.mxmoe_plan_layer(C.byref(ps["calls"][0]), C.byref(ps["calls"][1]), ps["recv"].data_ptr(), experts, ps["shared_rows"], stream))
    torch.cuda.synchronize()
    assert int(ps["recv"].sum()) == routed
    for k in ("recv", "row_of_slot"):
        assert torch.equal(ps[k], snap[k]), k
    for k in ("dst", "perm", "slot"):                                    # rows past the routed ones are not written by either
        assert torch.equal(ps[k][:routed], snap[k][:routed]), k
    et = ps["et"]
    first, last = lib.mxmoe_plan_offset(1, et), lib.mxmoe_plan_offset(4, et) + 12 * et
    for now, before in zip((ps["b1"]["plan"], ps["b2"]["plan"]), plans):
        a, b = now.cpu().numpy(), before.cpu().numpy()
        assert np.array_equal(a[:56], b[:56])                               # the header's pointers (same buffers on both sides)
        ai, bi = a[56:].view(np.int32), b[56:].view(np.int32)               # offset, entries, tiles, phases; phase_tile0[9]; phase_wg0[9]; flat; entries
        ne, nph = int(bi[1]), int(bi[3])
        assert ne > 0 and np.array_equal(ai[:4], bi[:4]) and np.array_equal(ai[4:5 + nph], bi[4:5 + nph]) and np.array_equal(ai[13:14 + nph], bi[13:14 + nph])
        assert ai[22] == bi[22] and np.array_equal(ai[23:23 + 4 * ne], bi[23:23 + 4 * ne])
        assert np.array_equal(a[first:last], b[first:last])                 # table, pointer arrays, row counts, sizes


def test_single_block_planning_writes_what_the_paired_launch_writes():
    """mxmoe_plan_block (one block per launch) against mxmoe_plan_layer (both blocks of the layer in one launch): identical plan
    buffers for the same counts."""
    from mxmoe_amd import _lib, synth

    cfg, layer = _small_layer(num_shared=1)
    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    layer(hidden, ids, w)
    torch.cuda.synchronize()
    lib = _lib.load()
    ps = layer._planned_setup(cfg.tokens, cfg.topk)
    stream = torch.cuda.current_stream().cuda_stream
    for key, out_store in (("b1", ps["mid"]), ("b2", ps["out"])):
        b = ps[key]
        fresh = torch.zeros_like(b["plan"])
        _lib.check(lib, lib.mxmoe_plan_block(b["kid"], ps["recv"].data_ptr(), cfg.num_experts, ps["shared_rows"], b["d"].data_ptr(), b["h"], b["inp"].data_ptr(),
                                             b["scale"].data_ptr(), out_store.data_ptr(), fresh.data_ptr(), stream))
        torch.cuda.synchronize()
        got, want = fresh.cpu().numpy().copy(), b["plan"].cpu().numpy().copy()
        # the header holds pointers into its own plan buffer (As .. sizes): compare them relative to the buffer's address
        g64, w64 = got[:56].view(np.int64).copy(), want[:56].view(np.int64).copy()
        assert g64[5] == 0 and w64[5] == 0                                  # no accumulator dumps
        g64[5], w64[5] = fresh.data_ptr(), b["plan"].data_ptr()
        assert np.array_equal(g64 - fresh.data_ptr(), w64 - b["plan"].data_ptr())
        gi, wi = got[56:].view(np.int32), want[56:].view(np.int32)          # offset, entries, tiles, phases; phase_tile0[9]; phase_wg0[9]; flat; entries
        ne, nph = int(wi[1]), int(wi[3])
        assert np.array_equal(gi[:4], wi[:4]) and np.array_equal(gi[4:5 + nph], wi[4:5 + nph]) and np.array_equal(gi[13:14 + nph], wi[13:14 + nph])
        assert gi[22] == wi[22] and np.array_equal(gi[23:23 + 4 * ne], wi[23:23 + 4 * ne])
        first, last = lib.mxmoe_plan_offset(1, ps["et"]), lib.mxmoe_plan_offset(4, ps["et"]) + 12 * ps["et"]
        assert np.array_equal(got[first:last], want[first:last])             # table, pointer arrays, row counts, sizes (what follows is padding)


def test_combine_entry_points_of_the_planned_forward_agree():
    """mxmoe_combine_planned (inverse map from the permutation) against mxmoe_unpermute_combine_planned (inverse map built from
    src_slot by two preparation launches) on the same plan and down output, with dropped ids."""
    from mxmoe_amd import _lib

    cfg, layer = _small_layer(num_shared=1)
    from mxmoe_amd import synth

    hidden = synth.make_hidden(cfg)
    ids, w = synth.make_routing(cfg)
    ids = torch.where(ids == 2, torch.full_like(ids, cfg.num_experts + 3), ids)
    wd = w.to("cuda").contiguous()
    want = layer(hidden, ids, wd).clone()
    lib = _lib.load()
    ps = layer._planned_setup(cfg.tokens, cfg.topk)
    out = torch.zeros_like(want)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(lib, lib.mxmoe_unpermute_combine_planned(ps["out"].data_ptr(), ps["b2"]["plan"].data_ptr(), ps["et"], wd.data_ptr(), ps["slot"].data_ptr(), cfg.tokens,
                                                        cfg.topk, cfg.hidden, out.data_ptr(), ps["comb_ws"].data_ptr(), stream))
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_planned_forward_replays_from_a_graph():
    """The whole forward inside a HIP graph (nothing in it synchronises, allocates or depends on the routing): each replay, with new
    routing and new hidden states written into the captured input buffers and eager work in between, equals the eager forward."""
    from mxmoe_amd import synth

    cfg, layer = _small_layer(1)
    hidden = synth.make_hidden(cfg).cuda()
    ids, w = synth.make_routing(cfg)
    ids, w = ids.cuda(), w.cuda()
    out = torch.empty((cfg.tokens, cfg.hidden), dtype=torch.float16, device="cuda")
    layer(hidden, ids, w, out=out)                                      # first call: allocates the layer's buffers
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(hidden, ids, w, out=out)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer(hidden, ids, w, out=out)
    gen = torch.Generator(device="cpu")
    for replay in range(4):
        gen.manual_seed(100 + replay)
        new_ids = torch.stack([torch.randperm(cfg.num_experts, generator=gen)[: cfg.topk] for _ in range(cfg.tokens)]).to(torch.int32)
        if replay == 2:
            new_ids[:, :] = torch.tensor([1, 3], dtype=torch.int32)     # all tokens on two experts: other experts empty
        new_w = torch.rand(cfg.tokens, cfg.topk, generator=gen)
        new_h = torch.randn(cfg.tokens, cfg.hidden, generator=gen).half()
        layer.forward(new_h, new_ids)                                   # eager reference (and eager work between the replays)
        want = layer.combine(new_w).clone()
        hidden.copy_(new_h.cuda())
        ids.copy_(new_ids.cuda())
        w.copy_(new_w.cuda())
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"
    # the same through the layer's own capture object
    cap = layer.capture(cfg.tokens)
    for replay in range(2):
        gen.manual_seed(200 + replay)
        new_ids = torch.stack([torch.randperm(cfg.num_experts, generator=gen)[: cfg.topk] for _ in range(cfg.tokens)]).to(torch.int32)
        new_w = torch.rand(cfg.tokens, cfg.topk, generator=gen)
        new_h = torch.randn(cfg.tokens, cfg.hidden, generator=gen).half()
        layer.forward(new_h, new_ids)
        want = layer.combine(new_w).clone()
        cap.hidden.copy_(new_h.cuda())
        cap.topk_ids.copy_(new_ids.cuda())
        cap.topk_weights.copy_(new_w.cuda())
        torch.cuda.synchronize()
        got = cap.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"captured replay {replay}"
