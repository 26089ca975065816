"""Synthetic MoE layers of the five benchmark configurations (seeded, no datasets or checkpoints needed).

The reference derives its workloads from traced HF models (mxmoe/quant/moe_tracer.py:174-211 ->
mxmoe/kernels/gen_workload.py:31-103) which need network access; these generators produce layers of the same shapes:

  c1  Qwen1.5-MoE  fp16            T=512   E=60 top-4  K=2048 I=1408   Gaussian router
  c2  Qwen1.5-MoE  w4a4            T=8192  same layer, Hadamard-rotated per-token int4 activations
  c3  Qwen1.5-MoE  w4a4 / w8a8     T=8192  per-block 50/50 draw, Zipf(1.2) expert popularity (Gumbel top-k)
  c4  DS-V2-Lite   w4a16 / w3a16   T=32    E=64 top-6 + 2 shared experts, group-128 asymmetric, 30 % of blocks w3
  c5  Mixtral-8x7B w4a4/w8a8/w4a16 T=8192  E=8 top-2 K=4096 I=14336, router bias N(0, 0.5)

Seeds (torch.Generator on the CPU): weights 0, activations 1, router 2, format draw 3, routing bias 4.
"""
from __future__ import annotations

from dataclasses import dataclass, replace

import torch

W4A4 = (4, 4, -1, True)
W8A8 = (8, 8, -1, True)
FP16 = (16, 16, -1, True)
W4A16 = (16, 4, 128, False)
W3A16 = (16, 3, 128, False)
W2A16 = (16, 2, 128, False)
W4A4G128 = (4, 4, 128, True)


def qcfg_str(qp) -> str:
    a, w, g, s = qp
    if a >= 16 and w >= 16:
        return "fp16"
    return f"w{w}a{a}_g{g}_{'sym' if s else 'asym'}"


@dataclass
class MoEConfig:
    name: str
    model: str
    num_experts: int
    topk: int
    hidden: int          # K
    inter: int           # I (per expert)
    tokens: int
    num_shared: int = 0
    routing: str = "gaussian"      # gaussian | zipf | biased
    formats: tuple = (FP16,)
    format_probs: tuple = (1.0,)
    rotate: int = 0                # online Hadamard: 0 none, 1 rows of quantised experts, 2 all rows
    description: str = ""

    @property
    def rows(self) -> int:
        return self.tokens * self.topk


CONFIGS = {
    "c1": MoEConfig("c1", "qwen2_moe", 60, 4, 2048, 1408, 512, description="Qwen1.5-MoE fp16, 512 tokens"),
    "c2": MoEConfig("c2", "qwen2_moe", 60, 4, 2048, 1408, 8192, formats=(W4A4,), rotate=1, description="Qwen1.5-MoE uniform w4a4_g-1_sym, 8192 tokens"),
    "c3": MoEConfig("c3", "qwen2_moe", 60, 4, 2048, 1408, 8192, routing="zipf", formats=(W4A4, W8A8), format_probs=(0.5, 0.5), rotate=1,
                    description="Qwen1.5-MoE mixed w4a4/w8a8, Zipf(1.2) routing, 8192 tokens"),
    "c4": MoEConfig("c4", "ds2", 64, 6, 2048, 1408, 32, num_shared=2, formats=(W4A16, W3A16), format_probs=(0.7, 0.3),
                    description="DeepSeek-V2-Lite w4a16/w3a16 g128 asym, 32 tokens, 2 shared experts"),
    "c5": MoEConfig("c5", "mixtral", 8, 2, 4096, 14336, 8192, routing="biased", formats=(W4A4, W8A8, W4A16), format_probs=(0.4, 0.4, 0.2), rotate=1,
                    description="Mixtral-8x7B mixed w4a4/w8a8/w4a16_g128, 8192 tokens"),
}


def get_config(name: str, tokens: int | None = None) -> MoEConfig:
    cfg = CONFIGS[name]
    return replace(cfg, tokens=tokens) if tokens else cfg


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def make_hidden(cfg: MoEConfig) -> torch.Tensor:
    return torch.randn(cfg.tokens, cfg.hidden, generator=_gen(1), dtype=torch.float32).to(torch.float16)


def make_routing(cfg: MoEConfig):
    """(topk_ids int32 [T, k], topk_weights fp32 [T, k]): softmax -> top-k -> renormalise (mxmoe/quant/moe_tracer.py:79-86)."""
    g = _gen(2)
    e = cfg.num_experts
    if cfg.routing == "zipf":
        # expert popularity ~ rank^-1.2; each token draws topk DISTINCT experts by Gumbel top-k on log p
        p = torch.arange(1, e + 1, dtype=torch.float64) ** -1.2
        logp = (p / p.sum()).log().to(torch.float32)
        u = torch.rand(cfg.tokens, e, generator=g, dtype=torch.float32).clamp_(1e-20, 1.0)
        logits = logp + (-(-u.log()).log())
    else:
        logits = torch.randn(cfg.tokens, e, generator=g, dtype=torch.float32)
        if cfg.routing == "biased":
            logits = logits + 0.5 * torch.randn(e, generator=_gen(4), dtype=torch.float32)
    probs = torch.softmax(logits, dim=1, dtype=torch.float32)
    w, ids = torch.topk(probs, cfg.topk, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return ids.to(torch.int32), w


def draw_formats(cfg: MoEConfig):
    """Per expert (incl. the shared one as index E): (gate_up qparams, down qparams); gate and up share a format
    (the ILP enforces it, mxmoe/quant/bits_solver.py:378-379)."""
    g = _gen(3)
    n = cfg.num_experts + (1 if cfg.num_shared else 0)
    probs = torch.tensor(cfg.format_probs, dtype=torch.float64)
    draw = torch.multinomial(probs, 2 * n, replacement=True, generator=g).reshape(n, 2)
    return [(cfg.formats[int(draw[i, 0])], cfg.formats[int(draw[i, 1])]) for i in range(n)]


def expert_weights(cfg: MoEConfig, e: int):
    """fp16 N(0, 0.02) weights of expert e: (W13 [2I, K] = [gate; up], W2 [K, I]).  Index E is the fused shared expert
    with intermediate size I * num_shared."""
    g = _gen(1000 + e)  # derived from the weight seed 0, one stream per expert so experts can be made lazily
    i = cfg.inter * (cfg.num_shared if e == cfg.num_experts else 1)
    w13 = (torch.randn(2 * i, cfg.hidden, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    w2 = (torch.randn(cfg.hidden, i, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    return w13, w2


def qconfig_dict(cfg: MoEConfig, layer: int = 0) -> dict:
    """The reference's qconfig JSON (mxmoe/kernels/qconfig.py:66-80) for this configuration."""
    experts = {}
    for e, (gu, dn) in enumerate(draw_formats(cfg)):
        def lin(qp):
            a, w, gs, s = qp
            return {"w_bits": w, "w_gsize": gs, "w_sym": s, "w_clip": [1.0, 1.0], "a_bits": a, "a_gsize": -1, "a_sym": True, "a_clip": [1.0, 1.0]}
        experts[str(e)] = {"gate": lin(gu), "up": lin(gu), "down": lin(dn)}
    return {str(layer): {"experts": experts}}


def trace_dict(cfg: MoEConfig, layer: int = 0) -> dict:
    """The reference's gate-trace JSON (mxmoe/quant/moe_tracer.py:189-206) for this configuration's routing."""
    ids, _ = make_routing(cfg)
    freq = torch.bincount(ids.reshape(-1).to(torch.int64), minlength=cfg.num_experts).tolist()
    return {"topk": cfg.topk, "NK": [cfg.inter, cfg.hidden], "num_tokens": cfg.tokens, "num_shared_experts": cfg.num_shared, f"layer-{layer}": {"access_freq": freq}}
