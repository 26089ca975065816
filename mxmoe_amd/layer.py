"""One mixed-precision MoE MLP layer on the GPU: permute + quantise, fused gate_up GroupGEMM, SiLU*up + quantise,
fused down GroupGEMM.  This is the sequence a caller of the reference's `mxmoe_ops` runs
(mxmoe/kernels/src/ref_bind.cu: quant_inp_act :434, gg_mxmoe_share_fused :312, silu_mul_then_quant :595, gg_mxmoe_share_fused again),
packaged so the pointer tables of both launches are built once and every later step is launch-only.
"""
from __future__ import annotations

import torch

from . import ops
from .synth import MoEConfig, draw_formats, expert_weights
from .weights import quantize_and_pack


class MxMoELayer:
    def __init__(self, cfg: MoEConfig, device="cuda", formats=None, weights=None, keep_codes: bool = False, packed=None):
        """weights: [(W13, W2)] fp16 per expert (default: the configuration's seeded synthetic weights); packed: ([PackedWeight] for
        gate_up, [PackedWeight] for down) already quantised and packed, e.g. from `checkpoint.load_layer` (formats are taken from them)."""
        self.cfg = cfg
        self.device = torch.device(device)
        self.n_exp_total = cfg.num_experts + (1 if cfg.num_shared else 0)
        if packed is not None:
            self.w13, self.w2 = list(packed[0]), list(packed[1])
            assert len(self.w13) == len(self.w2) == self.n_exp_total, "one packed gate_up and down block per expert (shared expert last)"
            for w in self.w13 + self.w2:
                w.data = w.data.to(self.device)
                w.scale = None if w.scale is None else w.scale.to(self.device)
            self.formats = [(tuple(a.qparams), tuple(b.qparams)) for a, b in zip(self.w13, self.w2)]
        else:
            self.formats = formats or draw_formats(cfg)
            self.w13, self.w2 = [], []
        for e in range(self.n_exp_total if packed is None else 0):
            w13, w2 = weights[e] if weights is not None else expert_weights(cfg, e)
            gu, dn = self.formats[e]
            self.w13.append(quantize_and_pack(w13.to(self.device), gu, keep_codes))
            self.w2.append(quantize_and_pack(w2.to(self.device), dn, keep_codes))
        self.qp_gate_up = [f[0] for f in self.formats]
        self.qp_down = [f[1] for f in self.formats]
        self.state = None

    @property
    def weight_bytes(self) -> int:
        return sum(w.nbytes for w in self.w13) + sum(w.nbytes for w in self.w2)

    # ---- the four steps -------------------------------------------------------------------------------------
    def prepare(self, hidden: torch.Tensor, topk_ids: torch.Tensor, dump_acc: bool = False):
        """Run the prologue once and build both launch plans; returns self.state (buffers + plans)."""
        cfg = self.cfg
        hidden = hidden.to(self.device)
        topk_ids = topk_ids.to(self.device)
        st = {}
        (st["inp"], st["sa"], st["mid"], st["inp_store"], st["sa_store"], st["mid_store"], st["recv"], st["perm"], st["dst"]) = ops.quant_inp_act(
            hidden, topk_ids, cfg.num_experts, cfg.inter, cfg.num_shared, self.qp_gate_up, rotate=cfg.rotate)
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        acc1 = [torch.zeros(m.shape, dtype=torch.int32, device=self.device) for m in st["mid"]] if dump_acc else None
        st["gg1"] = ops.prepare_gg(st["inp"], [w.data for w in self.w13], st["sa"], [w.scale for w in self.w13], st["mid"], 2 * cfg.inter, cfg.hidden,
                                   2 * i_sh, cfg.hidden, self.qp_gate_up, st["recv"], acc_dump=acc1)
        st["acc1"] = acc1
        st["dump_acc"] = dump_acc
        st["hidden"], st["topk_ids"] = hidden, topk_ids
        self.state = st
        return st

    def gate_up(self):
        self.state["gg1"].run()

    def act(self):
        cfg, st = self.cfg, self.state
        (st["inp2"], st["sa2"], st["out"], st["inp2_store"], st["sa2_store"], st["out_store"]) = ops.silu_mul_then_quant(
            st["mid_store"], len(st["mid"]), cfg.num_experts, cfg.hidden, cfg.inter, cfg.num_shared, cfg.tokens, cfg.topk, st["dst"], st["recv"],
            self.qp_down, rotate=cfg.rotate)
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        acc2 = [torch.zeros(o.shape, dtype=torch.int32, device=self.device) for o in st["out"]] if st["dump_acc"] else None
        st["gg2"] = ops.prepare_gg(st["inp2"], [w.data for w in self.w2], st["sa2"], [w.scale for w in self.w2], st["out"], cfg.hidden, cfg.inter,
                                   cfg.hidden, i_sh, self.qp_down, st["recv"], acc_dump=acc2)
        st["acc2"] = acc2

    def down(self):
        self.state["gg2"].run()

    def combine(self, topk_weights: torch.Tensor) -> torch.Tensor:
        """Un-permute and mix the down outputs back into token order: [T, K] fp16."""
        cfg, st = self.cfg, self.state
        st["final"] = ops.gg_unpermute_out(st["out_store"], st["topk_ids"], topk_weights.to(self.device), cfg.num_experts, cfg.hidden, cfg.num_shared)
        return st["final"]

    def forward(self, hidden, topk_ids, dump_acc: bool = False):
        """Full layer up to the per-problem down-projection outputs (list of [M_p, K] fp16, sorted-by-expert rows)."""
        self.prepare(hidden, topk_ids, dump_acc)
        self.gate_up()
        self.act()
        self.down()
        return self.state["out"]

    def __call__(self, hidden: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor) -> torch.Tensor:
        """The whole MoE MLP, `(hidden [T, K] fp16, topk_ids [T, k] int32, topk_weights [T, k] fp32) -> [T, K] fp16`: what a serving
        framework's fused-MoE operator computes after routing (permute, quantise, gate_up, SiLU * up, down, un-permute + combine)."""
        self.forward(hidden, topk_ids)
        return self.combine(topk_weights)

    # ---- accounting -----------------------------------------------------------------------------------------
    def gemm_ops(self) -> int:
        st = self.state
        return st["gg1"].ops + st["gg2"].ops

    def algorithmic_bytes(self) -> dict:
        """Bytes every launch must move at least once: packed weights + scales of touched experts, packed activations
        + their scales, fp16 outputs."""
        st = self.state
        recv = st["recv"]
        cfg = self.cfg
        touched = [e for e in range(self.n_exp_total) if e == cfg.num_experts or int(recv[e]) > 0]
        out = {}
        for name, ws, a_list, s_list, c_list in (("gate_up", self.w13, st["inp"], st["sa"], st["mid"]), ("down", self.w2, st["inp2"], st["sa2"], st["out"])):
            w = sum(ws[e].nbytes for e in touched)
            a = sum(t.numel() * t.element_size() for t in a_list) + sum(t.numel() * t.element_size() for t in s_list)
            c = sum(t.numel() * t.element_size() for t in c_list)
            out[name] = {"weights": w, "activations": a, "outputs": c, "total": w + a + c}
        return out
