"""One mixed-precision MoE MLP layer on the GPU: permute + quantise, fused gate_up GroupGEMM, SiLU*up + quantise,
fused down GroupGEMM.  This is the sequence a caller of the reference's `mxmoe_ops` runs
(mxmoe/kernels/src/ref_bind.cu: quant_inp_act :434, gg_mxmoe_share_fused :312, silu_mul_then_quant :595, gg_mxmoe_share_fused again),
packaged so the pointer tables of both launches are built once and every later step is launch-only.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib, ops
from . import layer_tables as LT
from .hadamard import device_signs
from .synth import MoEConfig, draw_formats, expert_weights
from .weights import quantize_and_pack


class MxMoELayer:
    def __init__(self, cfg: MoEConfig, device="cuda", formats=None, weights=None, keep_codes: bool = False, packed=None, bf6: bool = False, fp8: bool = False):
        """weights: [(W13, W2)] fp16 per expert (default: the configuration's seeded synthetic weights); packed: ([PackedWeight] for
        gate_up, [PackedWeight] for down) already quantised and packed, e.g. from `checkpoint.load_layer` (formats are taken from them).
        bf6: run the w4a4 blocks on the 6-bit float matrix path: their weights are packed as bf6 fragments, the quantisers write their
        activations as bf6 fragments (tag 4) and the launch uses a kernel whose w4a4 tiles take that layout.  Same integer codes, same
        accumulators and outputs, bit for bit; the operands occupy 0.75 instead of 0.5 bytes per value.  One flag for both linear
        blocks, or a pair (gate_up, down).
        fp8: run the w8a8 blocks in fp8 (OCP e4m3 codes for weights and activations, fp32 accumulation on the fp8 matrix instruction;
        the reference's w8a8_g-1_sym_E4M3) instead of int8.  A different number format: results differ from the int8 layer's."""
        self.cfg = cfg
        self.fp8 = bool(fp8)
        self.bf6_gate_up, self.bf6_down = (bool(bf6[0]), bool(bf6[1])) if isinstance(bf6, (tuple, list)) else (bool(bf6), bool(bf6))
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
            self.w13.append(quantize_and_pack(w13.to(self.device), gu, keep_codes, bf6=self.bf6_gate_up, fp8=self.fp8))
            self.w2.append(quantize_and_pack(w2.to(self.device), dn, keep_codes, bf6=self.bf6_down, fp8=self.fp8))
        self.qp_gate_up = [f[0] for f in self.formats]
        self.qp_down = [f[1] for f in self.formats]
        self.kid_gate_up = ops.select_kernel(self.qp_gate_up, self.bf6_gate_up, self.fp8)
        self.kid_down = ops.select_kernel(self.qp_down, self.bf6_down, self.fp8)
        self.state = None
        self._static = None

    def _variants(self, bf6: bool) -> int:
        """The quantisers' variants bit: set when the block's expert table may hold tag 4 (bf6 fragments) or tag 5 (fp8)."""
        return ops.ROWS_VARIANTS if bf6 or self.fp8 else 0

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
            hidden, topk_ids, cfg.num_experts, cfg.inter, cfg.num_shared, self.qp_gate_up, rotate=cfg.rotate, bf6=self.bf6_gate_up, fp8=self.fp8)
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        acc1 = [torch.zeros(m.shape, dtype=torch.int32, device=self.device) for m in st["mid"]] if dump_acc else None
        st["gg1"] = ops.prepare_gg(st["inp"], [w.data for w in self.w13], st["sa"], [w.scale for w in self.w13], st["mid"], 2 * cfg.inter, cfg.hidden,
                                   2 * i_sh, cfg.hidden, self.qp_gate_up, st["recv"], kernel_id=self.kid_gate_up, acc_dump=acc1)
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
            self.qp_down, rotate=cfg.rotate, bf6=self.bf6_down, fp8=self.fp8)
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        acc2 = [torch.zeros(o.shape, dtype=torch.int32, device=self.device) for o in st["out"]] if st["dump_acc"] else None
        st["gg2"] = ops.prepare_gg(st["inp2"], [w.data for w in self.w2], st["sa2"], [w.scale for w in self.w2], st["out"], cfg.hidden, cfg.inter,
                                   cfg.hidden, i_sh, self.qp_down, st["recv"], kernel_id=self.kid_down, acc_dump=acc2)
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

    def _static_tables(self):
        """Per-expert constants of both linear blocks (formats, row lengths, weight addresses), built once."""
        if self._static is None:
            cfg = self.cfg
            sh = [cfg.num_shared] if cfg.num_shared else []
            i_sh = cfg.inter * max(cfg.num_shared, 1)
            gu_w = [cfg.hidden] * self.n_exp_total
            gu_n = [2 * cfg.inter] * cfg.num_experts + [2 * i_sh for _ in sh]
            dn_w = [cfg.inter] * cfg.num_experts + [i_sh for _ in sh]
            dn_n = [cfg.hidden] * self.n_exp_total

            def ptrs(ws):
                return [w.data.data_ptr() for w in ws], [0 if w.scale is None else w.scale.data_ptr() for w in ws]

            self._static = (LT.static_block(self.qp_gate_up, gu_w, gu_n, *ptrs(self.w13), bf6=self.bf6_gate_up, fp8=self.fp8),
                            LT.static_block(self.qp_down, dn_w, dn_n, *ptrs(self.w2), bf6=self.bf6_down, fp8=self.fp8))
        return self._static

    # ---- the forward that never waits for its routing ---------------------------------------------------------
    def _planned_setup(self, t: int, topk: int):
        """Everything of the planned forward that depends only on the layer and on (tokens, top-k): block descriptors on both sides,
        kernels, worst-case grids, plan buffers, and the stores sized for the worst case.  Built once and reused."""
        key = (t, topk)
        cache = self.__dict__.setdefault("_planned", {})
        if key in cache:
            return cache[key]
        cfg, dev, lib = self.cfg, self.device, _lib.load()
        e_cnt, has_shared = cfg.num_experts, cfg.num_shared > 0
        et = self.n_exp_total
        r_cap = t * topk
        shared_rows = t if has_shared else 0
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        ps = {"r_cap": r_cap, "shared_rows": shared_rows, "et": et}

        def u8(n):
            return torch.empty(max(int(n), 16), dtype=torch.uint8, device=dev)

        def block(qps, ns, ks, ws, bf6):
            h = (_lib.BlockDesc * et)()
            for e in range(et):
                a, w, g, sym = qps[e]
                variant = 1 if bf6 and (int(a), int(w), int(g)) == (4, 4, -1) else (2 if self.fp8 and (int(a), int(w), int(g)) == (8, 8, -1) else 0)
                layout = (C.c_uint8 * 3)(variant, 0, 0)  # operand variant: 1 activations as bf6 fragments, 2 fp8 e4m3 codes
                h[e] = _lib.BlockDesc(int(a), int(w), int(g), 1 if sym else 0, layout, int(ns[e]), int(ks[e]), ws[e].data.data_ptr(),
                                      0 if ws[e].scale is None else ws[e].scale.data_ptr())
            d = torch.frombuffer(bytearray(bytes(h)), dtype=torch.uint8).to(dev)
            kid = lib.mxmoe_plan_select_kernel(-1, h, et)
            if kid < 0:
                raise RuntimeError(lib.mxmoe_last_error().decode())
            if t <= 64 and t * topk <= 12 * e_cnt:  # few tokens, and on average well under one 16-row tile per expert: a kernel made of 16-row few-token tiles alone, if one covers the formats
                few = lib.mxmoe_find_kernel(b"groupgemm_hz_fused_wo_skinny")
                if few >= 0 and lib.mxmoe_plan_select_kernel(few, h, et) == few:
                    kid = few
            grid = lib.mxmoe_plan_grid_bound(kid, h, e_cnt, r_cap, shared_rows)
            if grid < 0:
                raise RuntimeError(lib.mxmoe_last_error().decode())
            # worst-case stores: every routed row as wide as the widest routed expert's packed row
            tags = [ops.act_tag(int(q[0]), int(q[2]), bf6 and int(q[1]) == 4, self.fp8 and int(q[1]) == 8) for q in qps]
            # fp16 elements per row; bf6 fragments (tag 4) take 3/8 of an element per value and whole blocks of 32 rows per expert
            qld = [k * 3 // 8 if tg == 4 else (k if tg == 0 else (k // 2 if tg in (1, 5) else k // 4)) for tg, k in zip(tags, ks)]
            sld = [0 if tg == 0 else (k // 128 if tg == 3 else 1) for tg, k in zip(tags, ks)]
            sh = [e_cnt] if has_shared else []
            pad = 32 * e_cnt if 4 in tags else 0
            inp = 2 * (max(qld[:e_cnt]) * (r_cap + pad) + sum(qld[e] * (shared_rows + 31) // 32 * 32 for e in sh))
            sc = 2 * (max(sld[:e_cnt]) * r_cap + sum(sld[e] * shared_rows for e in sh))
            out = 2 * (max(ns[:e_cnt]) * r_cap + sum(ns[e] * shared_rows for e in sh))
            return {"h": h, "d": d, "kid": kid, "grid": grid, "plan": u8(lib.mxmoe_plan_bytes(et)), "inp": u8(inp), "scale": u8(sc), "out_bytes": out}

        sh = [1] if has_shared else []
        b1 = block(self.qp_gate_up, [2 * cfg.inter] * e_cnt + [2 * i_sh for _ in sh], [cfg.hidden] * et, self.w13, self.bf6_gate_up)
        b2 = block(self.qp_down, [cfg.hidden] * et, [cfg.inter] * e_cnt + [i_sh for _ in sh], self.w2, self.bf6_down)
        ps["b1"], ps["b2"] = b1, b2
        ps["mid"], ps["out"] = u8(b1["out_bytes"]), u8(b2["out_bytes"])
        call = lambda b, out_store: _lib.PlanCall(b["kid"], b["d"].data_ptr(), C.cast(b["h"], C.c_void_p), b["inp"].data_ptr(), b["scale"].data_ptr(),  # noqa: E731
                                                  out_store.data_ptr(), b["plan"].data_ptr())
        ps["calls"] = (call(b1, ps["mid"]), call(b2, ps["out"]))
        ps["dst"] = torch.empty(r_cap, dtype=torch.int32, device=dev)
        ps["perm"] = torch.empty(r_cap, dtype=torch.int64, device=dev)
        ps["slot"] = torch.empty(r_cap, dtype=torch.int64, device=dev)
        ps["row_of_slot"] = torch.empty(r_cap, dtype=torch.int32, device=dev)
        ps["recv"] = torch.empty(e_cnt, dtype=torch.int64, device=dev)
        ps["perm_ws"] = u8(lib.mxmoe_permute_workspace_bytes(r_cap, e_cnt))
        ps["comb_ws"] = u8(lib.mxmoe_combine_workspace_bytes(t, topk))

        def signs(n, n_shared):
            if not cfg.rotate:
                return 1, 1, None, None
            hk, hf, sg = device_signs(n, dev)
            if has_shared and device_signs(n_shared, dev)[0] != hk:
                raise RuntimeError("routed and shared intermediate sizes need the same Hadamard order")
            return hk, hf, sg, None if sg is None else sg.data_ptr()

        ps["had1"], ps["had2"] = signs(cfg.hidden, cfg.hidden), signs(cfg.inter, i_sh)
        # power-of-two rows without operand variants: the prologue quantises a token once per format, not once per destination row
        ps["per_token"] = ops.per_token_prologue(cfg.hidden, topk) and not self._variants(self.bf6_gate_up)
        ps["table1"] = b1["plan"].data_ptr() + lib.mxmoe_plan_offset(1, et)
        cache[key] = ps
        return ps

    def __call__(self, hidden: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """The whole MoE MLP, `(hidden [T, K] fp16, topk_ids [T, k] int32, topk_weights [T, k] fp32) -> [T, K] fp16`: what a serving
        framework's fused-MoE operator computes after routing (permute, quantise, gate_up, SiLU * up, down, un-permute + combine).

        Same kernels and results as `forward` + `combine`, but nothing here waits for the routing: the tables of both launches are
        derived from the tokens-per-expert counts by a planning kernel on the device (`mxmoe_plan_layer`: both blocks in one launch), the stores and plan
        buffers are allocated once per (tokens, top-k) for the worst case, and every launch argument is independent of the data.
        The call only enqueues six kernels (seven when more than 256 (token, slot) pairs are permuted, nine beyond what `mxmoe_permute_plan_layer_ws` takes; no synchronisation, no allocation after the first call when `out` is given), so it can
        be captured into a HIP graph.  Intermediate buffers belong to the layer and are reused by the next call of the same shape."""
        cfg, dev = self.cfg, self.device
        lib = _lib.load()
        hidden = hidden.to(dev).contiguous()
        ids = topk_ids.to(dev).to(torch.int32).contiguous()
        w = topk_weights.to(dev).to(torch.float32).contiguous()
        t, k_hid = hidden.shape
        topk = ids.shape[1]
        assert hidden.dtype == torch.float16 and k_hid == cfg.hidden and w.shape == ids.shape
        e_cnt, has_shared = cfg.num_experts, int(cfg.num_shared > 0)
        ps = self._planned_setup(t, topk)
        b1, b2 = ps["b1"], ps["b2"]
        stream = torch.cuda.current_stream().cuda_stream
        final = out if out is not None else torch.empty((t, cfg.hidden), dtype=torch.float16, device=dev)
        assert final.shape == (t, cfg.hidden) and final.dtype == torch.float16 and final.is_contiguous()
        ck = lambda rc: _lib.check(lib, rc)  # noqa: E731
        if ps["r_cap"] <= 256:  # decode-sized batch: permutation and planning in one launch
            ck(lib.mxmoe_permute_plan_layer(ids.data_ptr(), t, topk, e_cnt, ps["dst"].data_ptr(), ps["perm"].data_ptr(), ps["slot"].data_ptr(), ps["recv"].data_ptr(),
                                            ps["row_of_slot"].data_ptr(), C.byref(ps["calls"][0]), C.byref(ps["calls"][1]), ps["shared_rows"], stream))
        elif -(-ps["r_cap"] // 256) * e_cnt <= 16384:  # count, then scatter and plan side by side in one launch
            ck(lib.mxmoe_permute_plan_layer_ws(ids.data_ptr(), t, topk, e_cnt, ps["dst"].data_ptr(), ps["perm"].data_ptr(), ps["slot"].data_ptr(), ps["recv"].data_ptr(),
                                               ps["row_of_slot"].data_ptr(), C.byref(ps["calls"][0]), C.byref(ps["calls"][1]), ps["shared_rows"],
                                               ps["perm_ws"].data_ptr(), stream))
        else:
            ck(lib.mxmoe_build_permutation_inv(ids.data_ptr(), t, topk, e_cnt, ps["dst"].data_ptr(), ps["perm"].data_ptr(), ps["slot"].data_ptr(), ps["recv"].data_ptr(),
                                               ps["row_of_slot"].data_ptr(), ps["perm_ws"].data_ptr(), stream))
            ck(lib.mxmoe_plan_layer(C.byref(ps["calls"][0]), C.byref(ps["calls"][1]), ps["recv"].data_ptr(), e_cnt, ps["shared_rows"], stream))
        hk, hf, _sg, sgp = ps["had1"]
        if ps["per_token"]:
            ck(lib.mxmoe_quant_act_tokens(hidden.data_ptr(), b1["inp"].data_ptr(), b1["scale"].data_ptr(), ids.data_ptr(), ps["row_of_slot"].data_ptr(), ps["table1"],
                                          cfg.hidden, t, topk, e_cnt, has_shared, cfg.rotate, stream))
        else:
            ck(lib.mxmoe_quant_act_planned(hidden.data_ptr(), b1["inp"].data_ptr(), b1["scale"].data_ptr(), ps["dst"].data_ptr(), ps["perm"].data_ptr(), b1["plan"].data_ptr(),
                                           cfg.hidden, ps["r_cap"], t, e_cnt, has_shared, cfg.rotate | self._variants(self.bf6_gate_up), hk, hf, sgp, stream))
        ck(lib.mxmoe_group_gemm_planned(b1["kid"], b1["plan"].data_ptr(), ps["et"], b1["grid"], stream))
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        hk, hf, _sg, sgp = ps["had2"]
        ck(lib.mxmoe_silu_mul_quant_planned(ps["mid"].data_ptr(), b1["plan"].data_ptr(), b2["inp"].data_ptr(), b2["scale"].data_ptr(), ps["dst"].data_ptr(), b2["plan"].data_ptr(),
                                            cfg.inter, i_sh, ps["r_cap"], t, e_cnt, has_shared, cfg.rotate | self._variants(self.bf6_down), hk, hf, sgp, stream))
        ck(lib.mxmoe_group_gemm_planned(b2["kid"], b2["plan"].data_ptr(), ps["et"], b2["grid"], stream))
        ck(lib.mxmoe_combine_planned(ps["out"].data_ptr(), b2["plan"].data_ptr(), ps["et"], w.data_ptr(), ps["row_of_slot"].data_ptr(), t, topk, cfg.hidden,
                                     final.data_ptr(), stream))
        return final

    def forward_from_logits(self, hidden: torch.Tensor, router_logits: torch.Tensor, topk: int | None = None, renormalise: bool = False,
                            out: torch.Tensor | None = None) -> torch.Tensor:
        """`(hidden [T, K] fp16, router_logits [T, E] fp16 / fp32 / bf16) -> [T, K] fp16`: the routing kernel (softmax, top-k, optional
        renormalisation: `mxmoe_route_topk`) in front of `__call__`.  The ids and weights land in buffers the layer keeps per shape,
        so this too enqueues kernels only and can be captured."""
        t = hidden.shape[0]
        topk = self.cfg.topk if topk is None else topk
        assert router_logits.shape == (t, self.cfg.num_experts)
        ps = self._planned_setup(t, topk)
        if "route_ids" not in ps:
            ps["route_ids"] = torch.empty((t, topk), dtype=torch.int32, device=self.device)
            ps["route_w"] = torch.empty((t, topk), dtype=torch.float32, device=self.device)
        ops.route_topk(router_logits.to(self.device), topk, renormalise, out_ids=ps["route_ids"], out_weights=ps["route_w"])
        return self(hidden, ps["route_ids"], ps["route_w"], out=out)

    def capture(self, tokens: int, topk: int | None = None, logits_dtype: torch.dtype | None = None, renormalise: bool = False) -> "CapturedForward":
        """The planned forward for a fixed (tokens, top-k) shape, captured into a HIP graph: write the inputs into the returned
        object's `hidden`, `topk_ids`, `topk_weights` tensors, call `replay()`, read `out`.  Nothing in the forward depends on the
        routing at enqueue time, so one capture serves every routing; a replay has no per-kernel launch gaps (decode-sized batches
        gain most: 0.105 against 0.12 ms for DeepSeek-V2-Lite at 32 tokens).  With `logits_dtype` the graph starts at the router's
        logits instead (`forward_from_logits`): the input is then `router_logits` [tokens, experts] of that dtype."""
        return CapturedForward(self, tokens, self.cfg.topk if topk is None else topk, logits_dtype, renormalise)

    def call_with_host_tables(self, hidden: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor) -> torch.Tensor:
        """The whole MoE MLP with the tables of both launches built on the HOST (what the reference's operators do), `(hidden [T, K] fp16, topk_ids [T, k] int32, topk_weights [T, k] fp32) -> [T, K] fp16`: what a serving
        framework's fused-MoE operator computes after routing (permute, quantise, gate_up, SiLU * up, down, un-permute + combine).

        Same kernels and results as `forward` + `combine`, but the host side is one pass: after the single device-to-host copy of
        the tokens-per-expert counts every table of both launches is computed with array arithmetic and sent in one copy."""
        cfg, dev = self.cfg, self.device
        lib = _lib.load()
        hidden = hidden.to(dev).contiguous()
        ids = topk_ids.to(dev).to(torch.int32).contiguous()
        w = topk_weights.to(dev).to(torch.float32).contiguous()
        t, k_hid = hidden.shape
        topk = ids.shape[1]
        assert hidden.dtype == torch.float16 and k_hid == cfg.hidden and w.shape == ids.shape
        e_cnt, has_shared = cfg.num_experts, cfg.num_shared > 0
        gu, dn = self._static_tables()
        dst, perm, slot, recv = ops.build_permutation(ids, e_cnt)
        rows = np.empty(self.n_exp_total, np.int64)
        rows[:e_cnt] = recv.cpu().numpy()                     # the one synchronisation of the forward (as ref_bind.cu:451)
        if has_shared:
            rows[e_cnt] = t
        routed = int(rows[:e_cnt].sum())
        t1, t2 = LT.block_tables(gu, rows), LT.block_tables(dn, rows)

        def f16(n):
            return torch.empty(max(n, 1), dtype=torch.float16, device=dev)

        inp1, sa1, mid = f16(t1.inp_total), f16(t1.scale_total), f16(t1.out_total)
        inp2, sa2, out = f16(t2.inp_total), f16(t2.scale_total), f16(t2.out_total)
        p1, s1, q1 = LT.launch_tables(gu, rows, t1, inp1.data_ptr(), sa1.data_ptr(), mid.data_ptr())
        p2, s2, q2 = LT.launch_tables(dn, rows, t2, inp2.data_ptr(), sa2.data_ptr(), out.data_ptr())
        staging, off = LT.pack_staging([t1.table, t2.table, p1, p2, s1, s2])
        d_tab = torch.from_numpy(staging).to(dev)
        base = d_tab.data_ptr()
        count = p1.shape[1]
        stream = torch.cuda.current_stream().cuda_stream
        final = torch.empty((t, cfg.hidden), dtype=torch.float16, device=dev)
        if count == 0:
            return final.zero_()

        def signs(n, n_shared):
            if not cfg.rotate:
                return 1, 1, None
            hk, hf, sg = device_signs(n, dev)
            if has_shared and device_signs(n_shared, dev)[0] != hk:
                raise RuntimeError("routed and shared intermediate sizes need the same Hadamard order")
            return hk, hf, None if sg is None else sg.data_ptr()

        def launch(ptr_off, sizes_off, h_sizes, h_q, kid):
            row = lambda i: base + ptr_off + i * count * 8  # noqa: E731
            _lib.check(lib, lib.mxmoe_group_gemm(kid, row(0), row(1), row(2), row(3), row(4), row(4), None, None, None, None, base + sizes_off,
                                                 h_sizes.ctypes.data_as(C.POINTER(_lib.Dim3)), None, h_q.ctypes.data_as(C.POINTER(_lib.QParams)), count, None, stream))

        hk, hf, sg = signs(cfg.hidden, cfg.hidden)
        _lib.check(lib, lib.mxmoe_quant_act(hidden.data_ptr(), inp1.data_ptr(), sa1.data_ptr(), dst.data_ptr(), perm.data_ptr(), base + off[0],
                                            cfg.hidden, routed, t, e_cnt, int(has_shared), cfg.rotate | self._variants(self.bf6_gate_up), hk, hf, sg, stream))
        launch(off[2], off[4], s1, q1, self.kid_gate_up)
        i_sh = cfg.inter * max(cfg.num_shared, 1)
        hk, hf, sg = signs(cfg.inter, i_sh)
        _lib.check(lib, lib.mxmoe_silu_mul_quant(mid.data_ptr(), mid.data_ptr() + routed * 2 * cfg.inter * 2, inp2.data_ptr(), sa2.data_ptr(), dst.data_ptr(), base + off[1],
                                                 cfg.inter, i_sh, routed, t, e_cnt, int(has_shared), cfg.rotate | self._variants(self.bf6_down), hk, hf, sg, stream))
        launch(off[3], off[5], s2, q2, self.kid_down)
        ws = torch.empty(lib.mxmoe_combine_workspace_bytes(t, topk), dtype=torch.uint8, device=dev)
        shared_ptr = out.data_ptr() + routed * cfg.hidden * 2 if has_shared else None
        _lib.check(lib, lib.mxmoe_unpermute_combine(out.data_ptr(), shared_ptr, w.data_ptr(), slot.data_ptr(), routed, t, topk, cfg.hidden, final.data_ptr(), ws.data_ptr(), stream))
        return final

    # ---- accounting -----------------------------------------------------------------------------------------
    def gemm_ops(self) -> int:
        st = self.state
        return st["gg1"].ops + st["gg2"].ops

    def algorithmic_bytes(self) -> dict:
        """Bytes every launch must move at least once: packed weights + scales of touched experts, packed activations
        + their scales, fp16 outputs.  Codes count at their format's width (int4: half a byte) whatever layout carries them: the bf6
        fragments of the 6-bit float path occupy 0.75 bytes per value, which shows in measured traffic, not here."""
        st = self.state
        recv = st["recv"]
        cfg = self.cfg
        out = {}
        for name, qps, ws in (("gate_up", self.qp_gate_up, self.w13), ("down", self.qp_down, self.w2)):
            w = a = c = 0
            for e in range(self.n_exp_total):
                m = cfg.tokens if e == cfg.num_experts else int(recv[e])
                if m == 0:
                    continue
                a_bits, w_bits, gsize, _sym = (int(v) for v in qps[e])
                n, k = ws[e].n, ws[e].k
                if w_bits >= 16:
                    w += 2 * n * k
                elif a_bits >= 16:                      # weight-only: codes + (scale, zero) per group
                    w += n * k * w_bits // 8 + 4 * n * (k // gsize if gsize > 0 else 1)
                else:                                   # codes + one scale per channel (and group)
                    w += n * k * w_bits // 8 + 2 * n * (k // gsize if gsize > 0 else 1)
                a += m * k * min(a_bits, 16) // 8 + (0 if a_bits >= 16 else 2 * m * (k // gsize if gsize > 0 else 1))
                c += 2 * m * n
            out[name] = {"weights": w, "activations": a, "outputs": c, "total": w + a + c}
        return out


class CapturedForward:
    """`MxMoELayer.__call__` for one shape as a HIP graph over static input and output tensors."""

    def __init__(self, layer: MxMoELayer, tokens: int, topk: int, logits_dtype: torch.dtype | None = None, renormalise: bool = False):
        dev = layer.device
        self.hidden = torch.zeros((tokens, layer.cfg.hidden), dtype=torch.float16, device=dev)
        self.out = torch.empty((tokens, layer.cfg.hidden), dtype=torch.float16, device=dev)
        if logits_dtype is None:
            self.topk_ids = torch.zeros((tokens, topk), dtype=torch.int32, device=dev)
            self.topk_weights = torch.zeros((tokens, topk), dtype=torch.float32, device=dev)
            run = lambda: layer(self.hidden, self.topk_ids, self.topk_weights, out=self.out)  # noqa: E731
        else:
            self.router_logits = torch.zeros((tokens, layer.cfg.num_experts), dtype=logits_dtype, device=dev)
            run = lambda: layer.forward_from_logits(self.hidden, self.router_logits, topk, renormalise, out=self.out)  # noqa: E731
        side = torch.cuda.Stream(device=dev)  # (default priority)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # one eager run: every buffer of this shape exists before the capture
            run()
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            run()
        self._layer = layer  # the graph's kernels read the layer's buffers

    def replay(self) -> torch.Tensor:
        self.graph.replay()
        return self.out
