"""Host tables of one MoE layer forward, computed with array arithmetic instead of per-expert Python objects.

The reference builds these inside its operators: the per-expert `{tag, first row, packed-input offset, scale offset}` table of
`quant_inp_act` / `silu_mul_then_quant` (mxmoe/kernels/src/ref_bind.cu:475-505, 635-671) and the five pointer arrays, sizes and
QParams of `moe_mxmoe_share_fused` (ref_bind.cu:362-404).  `ops.py` mirrors that operator by operator and hands back per-problem
tensor views; a layer that only needs the launches can take everything from the tokens-per-expert counts in one pass, which is
what this module does.  All offsets are in fp16 elements, as in the reference; pointers are byte addresses.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .ops import BF6_FRAGMENT_HALVES, act_tag


@dataclass
class BlockStatic:
    """What does not change between forwards for one linear block (gate_up or down) of every expert (shared expert last)."""
    tag: np.ndarray      # int64 [Et] activation format tag (ref_bind.cu:461-473)
    qld: np.ndarray      # int64 [Et] fp16 elements per packed activation row
    sld: np.ndarray      # int64 [Et] scales per activation row
    out_ld: np.ndarray   # int64 [Et] fp16 elements per output row
    n: np.ndarray        # int64 [Et] output channels
    k: np.ndarray        # int64 [Et] reduction length
    b_ptr: np.ndarray    # int64 [Et] packed weights
    sb_ptr: np.ndarray   # int64 [Et] weight scales (0: none)
    q: np.ndarray        # int32 [Et, 4] (a_bits, w_bits, gsize, sym) in the 16-byte QParams layout


def static_block(qparams, widths, ns, b_ptrs, sb_ptrs, bf6: bool = False, fp8: bool = False) -> BlockStatic:
    """`qparams[e]`, input width `widths[e]`, output channels `ns[e]`, weight and scale addresses per expert; `bf6`: per-token int4
    activations are bf6 fragments (tag 4); `fp8`: per-token 8-bit activations are fp8 e4m3 codes (tag 5)."""
    et = len(qparams)
    tag = np.empty(et, np.int64)
    qld = np.empty(et, np.int64)
    sld = np.empty(et, np.int64)
    for e, (a_bits, w_bits, g, _s) in enumerate(qparams):
        t = act_tag(int(a_bits), int(g), bf6 and int(w_bits) == 4, fp8 and int(w_bits) == 8)
        if t < 0:
            raise RuntimeError("quant type not supported")
        w = int(widths[e])
        if t == 3 and w % 128:
            raise RuntimeError(f"group-128 activations need a row length that is a multiple of 128, got {w}")
        tag[e] = t
        qld[e] = w if t == 0 else (w // 2 if t in (1, 5) else w // 4)     # (tag 4: unused, see block_tables)
        sld[e] = 0 if t == 0 else (w // 128 if t == 3 else 1)
    q = np.array([[int(a), int(w), int(g), 1 if s else 0] for (a, w, g, s) in qparams], dtype=np.int32).reshape(et, 4)
    n = np.asarray(ns, dtype=np.int64)
    return BlockStatic(tag, qld, sld, n.copy(), n, np.asarray(widths, dtype=np.int64), np.asarray(b_ptrs, dtype=np.int64), np.asarray(sb_ptrs, dtype=np.int64), q)


def _exclusive(x: np.ndarray) -> np.ndarray:
    out = np.zeros_like(x)
    np.cumsum(x[:-1], out=out[1:])
    return out


@dataclass
class BlockTables:
    table: np.ndarray     # int64 [4, Et]: tag, first row, packed-input offset, scale offset
    inp_total: int        # fp16 elements of the packed-input store
    scale_total: int
    out_off: np.ndarray   # int64 [Et] offset of each expert's output rows
    out_total: int


def block_tables(st: BlockStatic, rows: np.ndarray) -> BlockTables:
    """`rows[e]` = rows of expert e in this forward (the shared expert, if any, has one row per token)."""
    # tag 4: whole blocks of 32 rows, k / 64 fragments each
    inp = np.where(st.tag == 4, -(-rows // 32) * (st.k // 64) * BF6_FRAGMENT_HALVES, st.qld * rows)
    sc = st.sld * rows
    out = st.out_ld * rows
    table = np.stack([st.tag, _exclusive(rows), _exclusive(inp), _exclusive(sc)])
    return BlockTables(table, int(inp.sum()), int(sc.sum()), _exclusive(out), int(out.sum()))


def launch_tables(st: BlockStatic, rows: np.ndarray, bt: BlockTables, inp_ptr: int, scale_ptr: int, out_ptr: int):
    """Pointer arrays [6, P] (A, B, scale_a, scale_b, C, accumulator dump = 0), sizes uint32 [P, 3] and QParams int32 [P, 4] of the
    non-empty problems, in expert order (ref_bind.cu:362-371 skips experts without rows the same way)."""
    live = np.nonzero(rows > 0)[0]
    p = live.size
    ptrs = np.zeros((6, p), np.int64)
    ptrs[0] = inp_ptr + 2 * bt.table[2, live]
    ptrs[1] = st.b_ptr[live]
    ptrs[2] = np.where(st.sld[live] > 0, scale_ptr + 2 * bt.table[3, live], 0)
    ptrs[3] = st.sb_ptr[live]
    ptrs[4] = out_ptr + 2 * bt.out_off[live]
    sizes = np.stack([rows[live], st.n[live], st.k[live]], axis=1).astype(np.uint32)
    return ptrs, np.ascontiguousarray(sizes), np.ascontiguousarray(st.q[live])


def pack_staging(arrays):
    """Concatenate int64 / uint32 arrays into one int64 buffer (each part 8-byte aligned) -> (buffer, byte offset of each part)."""
    parts, offs, pos = [], [], 0
    for a in arrays:
        raw = np.ascontiguousarray(a).reshape(-1).view(np.uint8)
        pad = (-raw.size) % 8
        if pad:
            raw = np.concatenate([raw, np.zeros(pad, np.uint8)])
        offs.append(pos)
        parts.append(raw)
        pos += raw.size
    buf = np.concatenate(parts) if parts else np.zeros(0, np.uint8)
    return buf.view(np.int64), offs
