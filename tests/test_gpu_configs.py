"""The benchmark workloads at their real sizes on the GPU.

The CPU oracle cannot run a whole 8192-token layer in test time, so the full-size runs are checked through size-independent
properties: the int32 accumulators of whole experts against an exact integer product of the very codes the launch read
(fp64 matmul on the GPU: every partial sum is an integer far below 2^53), the complete oracle chain (permute, rotate, quantise,
integer GEMM, epilogue) on a slice of rows of sampled experts, row bookkeeping (every routed row lands in exactly one
problem), and the stated fp16 tolerance against fp32 products of the dequantised operands."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
F16 = np.float16


def _rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-6)


def _build(name, tokens=None, dump=True):
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.get_config(name, tokens)
    hidden = synth.make_hidden(cfg)
    ids, _ = synth.make_routing(cfg)
    layer = MxMoELayer(cfg, keep_codes=True)
    outs = layer.forward(hidden, ids, dump_acc=dump)
    torch.cuda.synchronize()
    recv = layer.state["recv"].numpy()
    # problem index of every expert that received rows (the shared expert, when present, is the last problem)
    prob_of, p = {}, 0
    for e in range(cfg.num_experts):
        if recv[e] > 0:
            prob_of[e] = p
            p += 1
    if cfg.num_shared:
        prob_of[cfg.num_experts] = p
        p += 1
    assert p == len(outs)
    return cfg, hidden, ids, layer, outs, recv, prob_of


def _codes(t, bits):
    from mxmoe_amd import pack

    raw = t.contiguous().view(torch.uint8)          # the per-problem views are typed fp16 (the reference's `half*` tables)
    return pack.unpack_int4_k(raw) if bits == 4 else raw.view(torch.int8)


def _exact_acc(a_codes, w_codes):
    return (a_codes.double() @ w_codes.double().T).to(torch.int32)


def _check_wxax_experts(cfg, hidden, ids, layer, recv, prob_of, experts, oracle_rows=32):
    st = layer.state
    _, perm, _, _ = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    starts = np.concatenate([[0], np.cumsum(recv)])
    h = hidden.numpy()
    for e in experts:
        p = prob_of[e]
        (a1, w1b, _, _), (a2, w2b, _, _) = layer.formats[e]
        # whole expert, both launches: exact integer product of the codes the kernels read
        assert torch.equal(_exact_acc(_codes(st["inp"][p], a1), layer.w13[e].q), st["acc1"][p]), f"gate_up accumulators, expert {e}"
        assert torch.equal(_exact_acc(_codes(st["inp2"][p], a2), layer.w2[e].q), st["acc2"][p]), f"down accumulators, expert {e}"
        # the oracle chain from the fp16 hidden states on the first rows of the expert
        m = min(int(recv[e]), oracle_rows)
        x = h[perm[starts[e]:starts[e] + m]]
        w13 = layer_weights(cfg, e)[0]
        mid_k, mid_f, acc1 = O.linear_block(x, w13, layer.formats[e][0], cfg.rotate >= 1)
        assert np.array_equal(st["acc1"][p][:m].cpu().numpy(), acc1), f"oracle gate_up accumulators, expert {e}"
        assert np.array_equal(st["mid"][p][:m].cpu().numpy().view(np.uint16), mid_k.view(np.uint16)), f"oracle gate_up fp16, expert {e}"
        assert _rel(mid_k, mid_f) <= 1e-2


def layer_weights(cfg, e):
    from mxmoe_amd import synth

    w13, w2 = synth.expert_weights(cfg, e)
    return w13.numpy(), w2.numpy()


def _one_call_equals_stepwise(cfg, hidden, ids, layer):
    """Size-independent property: the whole forward as one call gives the bits of the operator-by-operator forward + combine."""
    from mxmoe_amd import synth

    _, w = synth.make_routing(cfg)
    stepwise = layer.combine(w).clone()
    assert torch.equal(layer(hidden, ids, w), stepwise)
    assert stepwise.shape == (cfg.tokens, cfg.hidden) and bool(torch.isfinite(stepwise).all())


def test_c2_uniform_w4a4_full_size():
    cfg, hidden, ids, layer, outs, recv, prob_of = _build("c2")
    assert int(recv.sum()) == cfg.tokens * cfg.topk == sum(o.shape[0] for o in outs)
    assert all(o.shape == (int(recv[e]), cfg.hidden) for e, o in zip(sorted(prob_of), outs))
    _check_wxax_experts(cfg, hidden, ids, layer, recv, prob_of, [0, 31, 59])
    assert all(bool(torch.isfinite(o).all()) for o in outs)
    _one_call_equals_stepwise(cfg, hidden, ids, layer)


def test_c3_mixed_zipf_full_size():
    cfg, hidden, ids, layer, outs, recv, prob_of = _build("c3")
    assert int(recv.sum()) == cfg.tokens * cfg.topk
    busiest, quietest = int(np.argmax(recv)), int(np.argmin(np.where(recv > 0, recv, 1 << 30)))
    assert recv[busiest] > 1000 and recv[quietest] < 128            # the skew the workload is defined by
    fm = layer.formats
    want = {busiest, quietest}
    for a_bits in (4, 8):                                            # one expert of each gate_up format on top
        want.add(next(e for e in prob_of if e < cfg.num_experts and fm[e][0][0] == a_bits))
    _check_wxax_experts(cfg, hidden, ids, layer, recv, prob_of, sorted(want))
    assert {f[0][1] for f in fm} == {4, 8} and {f[1][1] for f in fm} == {4, 8}
    assert all(bool(torch.isfinite(o).all()) for o in outs)
    _one_call_equals_stepwise(cfg, hidden, ids, layer)


def test_c4_weight_only_decode_full_size():
    cfg, hidden, ids, layer, outs, recv, prob_of = _build("c4", dump=False)
    st = layer.state
    _, perm, _, _ = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    starts = np.concatenate([[0], np.cumsum(recv)])
    h = hidden.numpy()
    touched = [e for e in range(cfg.num_experts) if recv[e] > 0]
    for e in touched[:3] + touched[-2:] + [cfg.num_experts]:
        p = prob_of[e]
        x = h if e == cfg.num_experts else h[perm[starts[e]:starts[e + 1]]]
        w13, w2 = layer_weights(cfg, e)
        (_, b1, g1, s1), (_, b2, g2, s2) = layer.formats[e]
        mid = O.gemm_fakequant(x, O.fake_quant(w13, b1, g1, s1))
        assert _rel(st["mid"][p].cpu().numpy(), mid) <= 1e-2, f"gate_up, expert {e}"
        y = O.silu_mul(st["mid"][p].cpu().numpy())                  # from the GPU's own intermediate: isolates the down launch
        out = O.gemm_fakequant(y, O.fake_quant(w2, b2, g2, s2))
        assert _rel(outs[p].cpu().numpy(), out) <= 1e-2, f"down, expert {e}"
    assert {f[0][1] for f in layer.formats} == {3, 4}
    _one_call_equals_stepwise(cfg, hidden, ids, layer)


def test_c1_fp16_full_size():
    """fp16 GroupGEMM at full size against an fp32 matmul of the same fp16 operands computed by the GPU's BLAS library (the plain
    fp32 reference of a floating-point kernel; the oracle's `gemm_fp16` covers the small fp16 cases of test_gpu_group_gemm.py)."""
    cfg, hidden, ids, layer, outs, recv, prob_of = _build("c1", dump=False)
    st = layer.state
    _, perm, _, _ = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    starts = np.concatenate([[0], np.cumsum(recv)])
    for e in [e for e in range(cfg.num_experts) if recv[e] > 0][:3]:
        p = prob_of[e]
        rows = torch.from_numpy(perm[starts[e]:starts[e + 1]])
        x = hidden[rows].cuda().float()
        w13, w2 = (w.cuda().float() for w in layer_weights_t(cfg, e))
        mid = (x @ w13.T)
        assert _rel(st["mid"][p].float().cpu().numpy(), mid.cpu().numpy()) <= 1e-2
        g, u = st["mid"][p].float()[:, :cfg.inter], st["mid"][p].float()[:, cfg.inter:]
        y = (g * torch.sigmoid(g) * u).half().float()
        assert _rel(outs[p].float().cpu().numpy(), (y @ w2.T).cpu().numpy()) <= 1e-2
    _one_call_equals_stepwise(cfg, hidden, ids, layer)


def layer_weights_t(cfg, e):
    from mxmoe_amd import synth

    return synth.expert_weights(cfg, e)


def test_c5_shaped_layer_reduced():
    """Mixtral-shaped mix (w4a4 / w8a8 / w4a16 g128, biased routing, rotation with the 28-point factor) at a size the oracle can
    follow end to end: every expert against the full oracle chain."""
    from mxmoe_amd import synth

    from test_gpu_layer import _run

    cfg = synth.MoEConfig("c5r", "mixtral", 8, 2, 512, 1792, 256, routing="biased", formats=(synth.W4A4, synth.W8A8, synth.W4A16),
                          format_probs=(0.4, 0.4, 0.2), rotate=1)
    fm = synth.draw_formats(cfg)
    assert {f[0] for f in fm} | {f[1] for f in fm} == {synth.W4A4, synth.W8A8, synth.W4A16}
    for r in _run(cfg, fm):
        gu, dn = fm[r["e"]]
        if gu[0] < 16:
            assert np.array_equal(r["g_acc1"], r["acc1"]), f"gate_up accumulators, expert {r['e']}"
            assert np.array_equal(r["g_mid"].view(np.uint16), r["mid"].view(np.uint16)), f"gate_up fp16, expert {r['e']}"
        else:
            assert _rel(r["g_mid"], r["mid"]) <= 1e-2, f"gate_up, expert {r['e']}"
        if gu[0] < 16 and dn[0] < 16:
            assert np.array_equal(r["g_acc2"], r["acc2"]), f"down accumulators, expert {r['e']}"
            assert np.array_equal(r["g_out"].view(np.uint16), r["out"].view(np.uint16)), f"down fp16, expert {r['e']}"
        elif dn[0] < 16:
            # a weight-only gate_up agrees with the oracle to the tolerance only, and the int4 / int8 re-quantisation in front of
            # the down launch turns last-bit differences into whole code steps: follow the oracle from the GPU's own intermediate
            w2 = synth.expert_weights(cfg, r["e"])[1].numpy()
            out_k, _, acc2 = O.linear_block(O.silu_mul(r["g_mid"]), w2, dn, True)
            assert np.array_equal(r["g_acc2"], acc2), f"down accumulators, expert {r['e']}"
            assert np.array_equal(r["g_out"].view(np.uint16), out_k.view(np.uint16)), f"down fp16, expert {r['e']}"
        else:
            assert _rel(r["g_out"], r["out"]) <= 1e-2, f"down, expert {r['e']}"


def test_c5_full_size():
    """Mixtral at its own dimensions (K = 4096 / 14336, 8192 tokens): the largest accumulators of the five workloads and the grouped
    tile order of long-row problems, against exact products.  Per launch of each sampled expert: integer formats compare every
    int32 accumulator of the expert with the exact integer product of the codes the launch read, and the first rows with the
    complete oracle chain from the fp16 inputs; the weight-only block compares its first rows with the oracle's fake-quant
    product to max-abs-rel 1e-2."""
    cfg, hidden, ids, layer, outs, recv, prob_of = _build("c5")
    assert int(recv.sum()) == cfg.tokens * cfg.topk == sum(o.shape[0] for o in outs)
    st, fm = layer.state, layer.formats
    _, perm, _, _ = O.permute_by_expert(ids.numpy(), cfg.num_experts)
    starts = np.concatenate([[0], np.cumsum(recv)])
    h = hidden.numpy()
    busiest = int(np.argmax(recv))
    want = {busiest}
    want.add(next(e for e in prob_of if fm[e][0][0] == 4))           # a w4a4 gate_up
    want.add(next(e for e in prob_of if fm[e][0][0] == 8))           # a w8a8 gate_up
    want.add(next(e for e in prob_of if fm[e][1][0] == 4))           # a w4a4 down
    want.add(next(e for e in prob_of if fm[e][1][0] == 8))           # a w8a8 down
    want.add(next(e for e in prob_of if fm[e][0][0] >= 16))          # the weight-only gate_up
    rows_oracle = 16
    for e in sorted(want):
        p = prob_of[e]
        gu, dn = fm[e]
        m = min(int(recv[e]), rows_oracle)
        x = h[perm[starts[e]:starts[e] + m]]
        w13, w2 = layer_weights(cfg, e)
        if gu[0] < 16:
            assert torch.equal(_exact_acc(_codes(st["inp"][p], gu[0]), layer.w13[e].q), st["acc1"][p]), f"gate_up accumulators, expert {e}"
            mid_k, mid_f, acc1 = O.linear_block(x, w13, gu, cfg.rotate >= 1)
            assert np.array_equal(st["acc1"][p][:m].cpu().numpy(), acc1), f"oracle gate_up accumulators, expert {e}"
            assert np.array_equal(st["mid"][p][:m].cpu().numpy().view(np.uint16), mid_k.view(np.uint16)), f"oracle gate_up fp16, expert {e}"
            assert _rel(mid_k, mid_f) <= 1e-2
        else:
            mid = O.gemm_fakequant(x, O.fake_quant(w13, gu[1], gu[2], gu[3]))
            assert _rel(st["mid"][p][:m].cpu().numpy(), mid) <= 1e-2, f"weight-only gate_up, expert {e}"
        if dn[0] < 16:
            assert torch.equal(_exact_acc(_codes(st["inp2"][p], dn[0]), layer.w2[e].q), st["acc2"][p]), f"down accumulators, expert {e}"
            # the oracle's down block from the GPU's own intermediate rows (isolates the activation step and the down launch)
            out_k, out_f, acc2 = O.linear_block(O.silu_mul(st["mid"][p][:m].cpu().numpy()), w2, dn, cfg.rotate >= 1)
            assert np.array_equal(st["acc2"][p][:m].cpu().numpy(), acc2), f"oracle down accumulators, expert {e}"
            assert np.array_equal(outs[p][:m].cpu().numpy().view(np.uint16), out_k.view(np.uint16)), f"oracle down fp16, expert {e}"
            assert _rel(out_k, out_f) <= 1e-2
    assert {f[0] for f in fm} | {f[1] for f in fm} == {(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False)}
    assert all(bool(torch.isfinite(o).all()) for o in outs)


def test_c5_one_call_equals_stepwise_at_real_row_lengths():
    """Mixtral row lengths (4096 and 14336 = 28 x 512) with a tenth of the tokens: the one-call forward against the stepwise one."""
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.get_config("c5", 512)
    hidden = synth.make_hidden(cfg)
    ids, _ = synth.make_routing(cfg)
    layer = MxMoELayer(cfg)
    layer.forward(hidden, ids)
    _one_call_equals_stepwise(cfg, hidden, ids, layer)
