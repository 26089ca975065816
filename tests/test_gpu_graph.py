"""The two GroupGEMM launches of a layer inside a HIP graph: the launch path allocates nothing, synchronises nothing and carries its
tables in the kernel arguments, so it can be captured; every replay must reproduce the eager result."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_captured_launches_replay_the_eager_result():
    from mxmoe_amd import synth
    from mxmoe_amd.layer import MxMoELayer

    cfg = synth.MoEConfig("t", "test", 6, 2, 256, 1408, 96, num_shared=1, rotate=1)
    g = synth.W4A4G128
    fm = [(synth.W4A4, synth.W8A8), (synth.W8A8, synth.W4A4), (g, g), (synth.W4A16, synth.W3A16), (synth.FP16, synth.FP16), (synth.W4A4, synth.W4A4),
          (synth.W8A8, synth.W8A8)]
    hidden = synth.make_hidden(cfg)
    ids, _ = synth.make_routing(cfg)
    layer = MxMoELayer(cfg, formats=fm)
    layer.forward(hidden, ids)
    torch.cuda.synchronize()
    st = layer.state
    want_mid, want_out = st["mid_store"].clone(), st["out_store"].clone()
    g1, g2 = st["gg1"], st["gg2"]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                  # warm-up on the capture stream, as torch asks
        g1.run()
        g2.run()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        g1.run()
        g2.run()
    for replay in range(4):
        st["mid_store"].fill_(float("nan"))                        # eager work between the replays
        st["out_store"].fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(st["mid_store"].view(torch.int16), want_mid.view(torch.int16)), f"gate_up outputs, replay {replay}"
        assert torch.equal(st["out_store"].view(torch.int16), want_out.view(torch.int16)), f"down outputs, replay {replay}"
