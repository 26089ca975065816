"""Offline weight pipeline: rotation matrix against the oracle's transform, weight rotation, state_dict naming, file round trip."""
import numpy as np
import pytest
import torch

from mxmoe_amd import checkpoint as C
from mxmoe_amd import synth
from oracle import mxmoe_oracle as O


@pytest.mark.parametrize("n", [256, 1408, 3584])   # pure Sylvester, 176 x 8, 28 x 128
def test_rotation_matrix_is_the_online_transform(n):
    q = C.hadamard_matrix(n).numpy()
    assert np.allclose(q @ q.T, np.eye(n), atol=1e-12)
    x = np.random.default_rng(0).standard_normal((3, n)).astype(np.float16)
    want = O.online_hadamard(x).astype(np.float64)           # fp16 result of the transform the kernels implement
    got = x.astype(np.float64) @ q.T
    assert np.abs(got - want).max() <= 2e-3 * np.abs(want).max()


def test_rotated_weights_cancel_the_online_rotation():
    g = torch.Generator().manual_seed(0)
    w = (torch.randn(64, 1408, generator=g) * 0.02).half()
    x = torch.randn(5, 1408, generator=g).double()
    q = C.hadamard_matrix(1408)
    wr = C.rotate_input_weights(w)
    assert wr.dtype == torch.float16
    y, yr = x @ w.double().T, (x @ q.T) @ wr.double().T
    assert (y - yr).abs().max() <= 2e-3 * y.abs().max()       # fp16 rounding of the rotated weights only


@pytest.mark.parametrize("model_id,shared", [("qwen2_moe", True), ("ds2", True), ("mixtral", False)])
def test_state_dict_names(model_id, shared):
    E, K, I = 3, 64, 32
    lin = C.MOE_WEIGHT_NAME_MAP[model_id]
    mlp = C.MOE_MLP_NAME_MAP[model_id]
    sd = {}
    for e in range(E):
        sd[f"model.layers.2.{mlp}.experts.{e}.{lin['gate']}.weight"] = torch.full((I, K), float(e))
        sd[f"model.layers.2.{mlp}.experts.{e}.{lin['up']}.weight"] = torch.full((I, K), e + 0.5)
        sd[f"model.layers.2.{mlp}.experts.{e}.{lin['down']}.weight"] = torch.full((K, I), -float(e))
    if shared:
        for b, shape in (("gate", (2 * I, K)), ("up", (2 * I, K)), ("down", (K, 2 * I))):
            sd[f"model.layers.2.{mlp}.{C.SHARED_NAME[model_id]}.{lin[b]}.weight"] = torch.full(shape, 9.0)
    ex = C.experts_from_state_dict(sd, model_id, 2, E)
    assert len(ex) == E + (1 if shared else 0)
    w13, w2 = ex[1]
    assert w13.shape == (2 * I, K) and w2.shape == (K, I)
    assert float(w13[0, 0]) == 1.0 and float(w13[I, 0]) == 1.5 and float(w2[0, 0]) == -1.0   # [gate; up]
    if shared:
        assert ex[-1][0].shape == (4 * I, K) and ex[-1][1].shape == (K, 2 * I)


def test_file_round_trip(tmp_path):
    cfg = synth.MoEConfig("t", "qwen2_moe", 3, 2, 256, 128, 16, num_shared=2, formats=(synth.W4A4, synth.W8A8, synth.W4A16, synth.FP16),
                          format_probs=(0.25, 0.25, 0.25, 0.25), rotate=1)
    formats = [(synth.W4A4, synth.W8A8), (synth.W4A16, synth.W4A4), (synth.FP16, synth.W3A16), (synth.W8A8, synth.W8A8)]
    experts = [synth.expert_weights(cfg, e) for e in range(4)]
    tensors, meta = C.pack_layer(experts, formats, rotate=1, model="qwen2_moe", layer=5, num_shared=2)
    path = str(tmp_path / "layer5.safetensors")
    C.save_layer(path, tensors, meta)
    w13, w2, meta2 = C.load_layer(path, device="cpu")
    assert meta2 == meta and meta["num_experts"] == 3 and meta["hidden"] == 256 and meta["inter"] == 128
    assert [(tuple(a.qparams), tuple(b.qparams)) for a, b in zip(w13, w2)] == [tuple(map(tuple, f)) for f in formats]
    for e in range(4):
        assert torch.equal(w13[e].data, tensors[f"e{e}.w13.data"]) and torch.equal(w2[e].data, tensors[f"e{e}.w2.data"])
        assert (w13[e].scale is None) == (formats[e][0] == synth.FP16)
        assert (w13[e].n, w13[e].k, w2[e].n, w2[e].k) == (256 * (2 if e == 3 else 1), 256, 256, 128 * (2 if e == 3 else 1))
    # rotation was applied exactly where the block's activations are quantised: the fp16 block of expert 2 is stored as given
    assert torch.equal(w13[2].data, experts[2][0])
    assert not torch.equal(C.rotate_input_weights(experts[2][0]), experts[2][0])


def test_formats_from_qconfig():
    qc = synth.qconfig_dict(synth.get_config("c4"))["0"]
    cfg = synth.get_config("c4")
    fm = C.formats_from_qconfig(qc, cfg.num_experts, True)
    assert len(fm) == cfg.num_experts + 1
    assert fm[:cfg.num_experts] == [tuple(map(tuple, f)) for f in synth.draw_formats(cfg)][:cfg.num_experts]
    assert fm[-1][0] == fm[-1][1]                                 # the shared expert takes its "gate" format for both blocks
    bad = {"experts": {"0": dict(qc["experts"]["0"], up=dict(qc["experts"]["0"]["up"], w_bits=8))}}
    with pytest.raises(ValueError, match="gate and up"):
        C.formats_from_qconfig(bad, 1, False)


def _gptq_like(n, k, bits, gsize, sym, dtype, seed):
    """A weight matrix as a GPTQ run leaves it (gptq.py:21-25, 51-100): grid from the original min / max, codes moved off the
    nearest ones by the error compensation (here: +-1 on a fifth of them), value = scale * (q - zero) in fp32, stored in `dtype`.
    Half of the groups avoid their extreme codes, so min / max of the stored values are not the ends of the grid."""
    g_ = torch.Generator().manual_seed(seed)
    g = k if gsize == -1 else gsize
    w = (torch.randn(n, k, generator=g_) * 0.02).reshape(-1, g)
    maxq = (1 << bits) - 1
    lo, hi = w.amin(1, keepdim=True), w.amax(1, keepdim=True)
    if sym:
        m = torch.maximum(lo.abs(), hi.abs())
        scale, zero = 2 * m / maxq, torch.full_like(m, (maxq + 1) / 2)
    else:
        scale = (hi - lo) / maxq
        zero = (-lo / scale).round()
    q = (w / scale).round() + zero
    q = q + (torch.rand(q.shape, generator=g_) < 0.2) * torch.randint(-1, 2, q.shape, generator=g_)
    inner = (torch.arange(q.shape[0]) % 2 == 0)[:, None]
    q = torch.where(inner, q.clamp(1, maxq - 1), q.clamp(0, maxq))
    return (scale * (q - zero)).reshape(n, k).to(dtype), (q - zero).reshape(n, k), scale


@pytest.mark.parametrize("bits,gsize,sym", [(4, -1, True), (8, -1, True), (4, 128, False), (3, 128, False), (2, 128, False), (4, 128, True)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_recover_grid_of_fake_quantised_weights(bits, gsize, sym, dtype):
    n, k = 48, 512
    w, t_true, s_true = _gptq_like(n, k, bits, gsize, sym, dtype, seed=bits * 10 + (gsize > 0))
    q, scale, zp = C.recover_grid(w, bits, gsize, sym)
    g = k if gsize == -1 else gsize
    # the recovered codes are the true ones up to one constant per group (zero for symmetric grids)
    d = (q - t_true).reshape(-1, g)
    if bits == 8 and dtype == torch.bfloat16:                 # bf16 keeps 8 significant bits: neighbouring 8-bit codes can share a value
        assert int(d.abs().max()) <= 1
    else:
        assert torch.equal(d, d[:, :1].expand_as(d))
    if sym:
        assert int(d.abs().max()) <= (1 if dtype == torch.bfloat16 and bits == 8 else 0) and float(zp.abs().max()) == 0
    else:
        assert int(q.min()) == 0 and int(q.max()) <= (1 << bits) - 1
    # the scale is the true one to the precision the stored values carry (a group holds at most 2^bits distinct values, each with its
    # type's rounding), and the values come back to within the file's own storage rounding
    assert ((scale.double() - s_true.double()).abs() <= (2.0**-8 if dtype == torch.bfloat16 else 2.0**-10) * s_true.double()).all()
    back = (q.reshape(-1, g) * scale.double() + zp.double()).reshape(n, k)
    ulp = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    # (plus the fp16 rounding of the stored scale and zero point, each below 2^-11 of the group's largest value)
    assert ((back - w.double()).abs() <= 2 * ulp * w.double().abs() + 2.0**-10 * w.double().abs().max()).all()
    # min / max re-quantisation of the same matrix lands on another grid wherever the extreme codes are unused
    from mxmoe_amd.quant import quant_minmax

    q2, s2, z2 = quant_minmax(w.to(torch.float16), bits, gsize, sym)
    rtn = (q2.reshape(-1, g).double() * s2.double() + z2.double()).reshape(n, k)
    if bits < 8:
        assert (rtn - w.double()).abs().max() > 4 * (back - w.double()).abs().max()


def test_recover_grid_refuses_weights_off_any_grid():
    w = (torch.randn(4, 256, generator=torch.Generator().manual_seed(1)) * 0.02).half()
    with pytest.raises(ValueError, match="grid"):
        C.recover_grid(w, 4, 128, False)
    # constant and all-zero groups are grids of one level
    z = torch.zeros(2, 128, dtype=torch.float16)
    q, s, zp = C.recover_grid(z, 4, 128, False)
    assert int(q.abs().max()) == 0 and float(zp.abs().max()) == 0
    c = torch.full((2, 128), 0.25, dtype=torch.float16)
    q, s, zp = C.recover_grid(c, 4, 128, False)
    assert torch.equal((q * s + zp).half(), c)


def test_pack_layer_of_fake_quantised_weights_equals_packing_their_codes(tmp_path):
    from mxmoe_amd.weights import pack_codes

    w13, t13, _ = _gptq_like(64, 256, 4, -1, True, torch.bfloat16, 3)
    w2, t2, _ = _gptq_like(256, 128, 4, 128, False, torch.bfloat16, 4)
    formats = [(synth.W4A4, synth.W4A16)]
    tensors, meta = C.pack_layer([(w13, w2)], formats, rotate=1, fake_quant=True)
    q, s, zp = C.recover_grid(w13, 4, -1, True)
    want = pack_codes(q, s, zp, synth.W4A4, 64, 256)
    assert torch.equal(tensors["e0.w13.data"], want.data) and torch.equal(tensors["e0.w13.scale"], want.scale)
    assert torch.equal(q, t13)
    # saved with torch.save as a GPTQ run does, read back as tensors only
    path = str(tmp_path / "fq.pt")
    torch.save({"model.layers.0.mlp.experts.0.gate_proj.weight": w13[:32], "model.layers.0.mlp.experts.0.up_proj.weight": w13[32:],
                "model.layers.0.mlp.experts.0.down_proj.weight": w2}, path)
    sd = C.load_fake_quant_state_dict(path)
    (a13, a2), = C.experts_from_state_dict(sd, "qwen2_moe", 0, 1)
    assert torch.equal(a13, w13) and torch.equal(a2, w2)
