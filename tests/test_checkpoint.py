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
