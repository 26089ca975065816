"""GPU tests of the routing kernel (`mxmoe_route_topk`: softmax over the experts, top-k, optional renormalisation; the gate
arithmetic of mxmoe/quant/moe_tracer.py:79-86) against the oracle, and of the layer forward that starts at the router's logits."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
# float tolerance of the weights: exp and the sums are fp32 on both sides, each within an ulp or two of the exact value
RTOL = 1e-5


def _check(logits_t: torch.Tensor, k: int, renorm: bool):
    from mxmoe_amd import ops

    ids, w = ops.route_topk(logits_t.to(DEV), k, renorm)
    torch.cuda.synchronize()
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    x = logits_t.to(torch.float32).numpy()
    o_ids, o_w = O.route_topk(x, k, renormalise=renorm)
    assert ids.dtype == np.int32 and w.dtype == np.float32 and ids.shape == o_ids.shape == w.shape
    # every row holds k distinct experts in range, in order of decreasing weight
    assert (ids >= 0).all() and (ids < x.shape[1]).all()
    assert all(len(set(r)) == k for r in ids.tolist())
    assert (np.diff(w, axis=1) <= 0).all()
    # ids are compared where no two DIFFERENT logits give probabilities closer than the tolerance around the cut (equal logits
    # have equal probabilities on both sides and fall to the lower id on both)
    z = x - x.max(axis=1, keepdims=True)
    p = np.exp(z.astype(np.float64))
    p /= p.sum(axis=1, keepdims=True)
    ps = -np.sort(-p, axis=1)[:, :min(k + 1, x.shape[1])]
    xs = -np.sort(-x, axis=1)[:, :min(k + 1, x.shape[1])]
    gap = np.where(np.diff(xs, axis=1) == 0, np.inf, -np.diff(ps, axis=1) / np.maximum(ps[:, :-1], 1e-30))
    clear = (gap > 1e-6).all(axis=1) if gap.size else np.ones(len(x), bool)   # (a few fp32 ulps)
    assert clear.mean() >= 0.9
    assert np.array_equal(ids[clear], o_ids[clear])
    assert np.allclose(w[clear], o_w[clear], rtol=RTOL, atol=1e-30)
    if renorm:
        assert np.allclose(w.sum(axis=1), 1.0, atol=1e-6)
    return ids, w


@pytest.mark.parametrize("t,e,k", [(1, 1, 1), (3, 8, 2), (97, 60, 4), (130, 64, 6), (33, 65, 8), (50, 160, 6), (21, 256, 8), (9, 4096, 8), (5, 100, 64)])
@pytest.mark.parametrize("renorm", [False, True])
def test_route_topk_matches_the_oracle(t, e, k, renorm):
    g = torch.Generator().manual_seed(100 * e + k)
    logits = torch.randn(t, e, generator=g, dtype=torch.float32) * 2.5
    _check(logits, k, renorm)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_route_topk_half_precision_logits_with_equal_values(dtype):
    """fp16 / bf16 logits are widened exactly; many of them collide, and equal probabilities go to the lower expert id."""
    g = torch.Generator().manual_seed(7)
    logits = (torch.randn(300, 60, generator=g) * 1.5).to(dtype)
    assert any(len(set(r)) < 60 for r in logits.to(torch.float32).tolist())  # there are equal logits inside rows
    _check(logits, 4, True)
    _check(logits, 6, False)


def test_route_topk_degenerate_rows():
    from mxmoe_amd import ops

    # all logits equal: experts 0 .. k-1, weight 1 / E each (1 / k renormalised)
    ids, w = ops.route_topk(torch.full((5, 12), 3.25, device=DEV), 3, False)
    assert ids.cpu().tolist() == [[0, 1, 2]] * 5 and np.allclose(w.cpu().numpy(), 1 / 12, rtol=1e-6)
    ids, w = ops.route_topk(torch.full((5, 12), -7.0, device=DEV), 3, True)
    assert ids.cpu().tolist() == [[0, 1, 2]] * 5 and np.allclose(w.cpu().numpy(), 1 / 3, rtol=1e-6)
    # experts switched off by a very negative logit have probability 0 and are taken last, in index order
    x = torch.full((2, 6), -1e9)
    x[:, 4] = 1.0
    x[:, 1] = 0.0
    ids, w = ops.route_topk(x.to(DEV), 4, False)
    assert ids.cpu().tolist() == [[4, 1, 0, 2]] * 2
    e = np.exp(-1.0)
    assert np.allclose(w.cpu().numpy(), [[1 / (1 + e), e / (1 + e), 0, 0]] * 2, rtol=1e-6)
    # hand-computed: probabilities 0.1, 0.4, 0.2, 0.3
    x = (torch.log(torch.tensor([[1.0, 4.0, 2.0, 3.0]])) - 2.0).to(DEV)
    ids, w = ops.route_topk(x, 2, True)
    assert ids.cpu().tolist() == [[1, 3]] and np.allclose(w.cpu().numpy(), [[4 / 7, 3 / 7]], rtol=1e-6)
    # results written into the caller's tensors
    oi = torch.full((1, 2), -5, dtype=torch.int32, device=DEV)
    ow = torch.zeros((1, 2), dtype=torch.float32, device=DEV)
    ri, rw = ops.route_topk(x, 2, False, out_ids=oi, out_weights=ow)
    assert ri is oi and rw is ow and oi.cpu().tolist() == [[1, 3]] and np.allclose(ow.cpu().numpy(), [[0.4, 0.3]], rtol=1e-6)
    with pytest.raises(ValueError):
        ops.route_topk(x.to(torch.float64), 2)
    with pytest.raises(RuntimeError):
        ops.route_topk(x, 5)


@pytest.mark.parametrize("tokens", [24, 300])
def test_forward_from_logits_equals_the_forward_from_ids(tokens):
    """`forward_from_logits` = routing kernel + the planned forward: the same bytes as the forward called with the routing kernel's
    own ids and weights, eagerly and from a HIP graph that starts at the logits (replayed with two routings)."""
    from mxmoe_amd import ops, synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("route", "test", 8, 2, 256, 512, tokens, num_shared=1, rotate=1)
    fm = [(synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4)] * 4 + [(synth.W8A8, synth.W8A8)]
    layer = MxMoELayer(cfg, formats=fm)
    hidden = synth.make_hidden(cfg).to(DEV)
    cap = layer.capture(tokens, logits_dtype=torch.float32, renormalise=True)
    for seed in (1, 2):
        g = torch.Generator().manual_seed(seed)
        logits = torch.randn(tokens, cfg.num_experts, generator=g).to(DEV)
        ids, w = ops.route_topk(logits, cfg.topk, True)
        o_ids, _ = O.route_topk(logits.cpu().numpy(), cfg.topk, True)
        assert np.array_equal(ids.cpu().numpy(), o_ids)
        want = layer(hidden, ids, w).clone()
        got = layer.forward_from_logits(hidden, logits, renormalise=True).clone()
        cap.hidden.copy_(hidden)
        cap.router_logits.copy_(logits)
        rep = cap.replay().clone()
        torch.cuda.synchronize()
        assert torch.isfinite(want.float()).all() and want.abs().max() > 0
        assert torch.equal(got, want) and torch.equal(rep, want)
