"""The five operators of the reference's `mxmoe_ops` extension (mxmoe/kernels/src/ref_bind.cu:759-768), same names,
argument order and return tuples, running on the gfx950 kernels behind the C-ABI.

Differences a caller can see, all deliberate:
  * rows of one expert keep their original (token, slot) order (the reference's torch::sort is unstable);
  * packed activations use this library's layouts (int4: two values per byte, even element in the low nibble);
  * failures raise RuntimeError instead of exit(EXIT_FAILURE) (mxmoe/kernels/src/include/helper.h:186-193);
  * `quant_inp_act` / `silu_mul_then_quant` accept `rotate=` (0 none, 1 rows of quantised experts, 2 all rows) for the
    online Hadamard rotation that the reference applies from Python (mxmoe/quant/rotation.py:403-421).
"""
from __future__ import annotations

import torch

from . import _lib
from .group_gemm import GroupGemmLaunch
from .hadamard import device_signs


def _stream():
    return torch.cuda.current_stream().cuda_stream


def act_tag(a_bits: int, gsize: int, bf6: bool = False, fp8: bool = False) -> int:
    """ref_bind.cu:461-473, plus two tags for operand variants that QParams cannot name: with `bf6`, per-token int4 codes are written
    as bf6 fragments (tag 4: the operand layout of the kernels whose w4a4 tiles run on the 6-bit float matrix path); with `fp8`,
    per-token 8-bit codes are fp8 e4m3 numbers instead of int8 ones (tag 5: for the kernels whose w8a8 tiles run the fp8 instruction,
    the reference's w8a8_g-1_sym_E4M3).  `select_kernel(..., bf6=, fp8=)` finds the matching kernel."""
    if a_bits >= 16:
        return 0
    if a_bits == 8 and gsize == -1:
        return 5 if fp8 else 1
    if a_bits == 4 and gsize == -1:
        return 4 if bf6 else 2
    if a_bits == 4 and gsize == 128:
        return 3
    return -1


BF6_FRAGMENT_HALVES = 768
ROWS_VARIANTS = 4         # bit 2 of the quantisers' `rotate` argument: the expert table may hold tags 4 (bf6 fragments) and 5 (fp8)      # fp16 elements of one 32-row x 64-k fragment (1536 bytes)


def packed_elems(tag: int, rows: int, width: int) -> int:
    """fp16 elements that `rows` packed activation rows of `width` values occupy (ref_bind.cu:491; tag 4: whole blocks of 32 rows)."""
    if tag == 4:
        return -(-rows // 32) * (width // 64) * BF6_FRAGMENT_HALVES
    return rows * (width if tag == 0 else (width // 2 if tag in (1, 5) else width // 4))


def kernel_variants(lib, kid: int) -> dict:
    """{format id: operand variant} of kernel `kid`'s branches that take a variant (1 bf6 fragments, 2 fp8 e4m3 codes, 3 bfloat16)."""
    import ctypes as C

    out, res = (C.c_int32 * 8)(), {}
    for b in range(lib.mxmoe_kernel_num_branches(kid)):
        lib.mxmoe_kernel_branch(kid, b, out)
        if out[0] >> 8:
            res[out[0] & 255] = out[0] >> 8
    return res


def select_kernel(qparams, bf6: bool = False, fp8: bool = False, lib=None, bf16: bool = False) -> int:
    """Registry index of the first fused kernel with a tile for every format in `qparams` whose operand variants are exactly the ones
    asked for: w4a4 operands as bf6 fragments (`bf6`), w8a8 operands as fp8 e4m3 codes (`fp8`), 16-bit float problems in bfloat16
    (`bf16`).  -1 (the launcher's own choice) when none is asked for; kernels with variants are never chosen automatically, since the
    launcher cannot see what the operands hold."""
    lib = lib or _lib.load()
    qs = sorted({tuple(int(v) for v in q) for q in qparams})
    want = {}
    if bf6 and (4, 4, -1, 1) in qs:
        want[2] = 1
    if fp8 and (8, 8, -1, 1) in qs:
        want[1] = 2
    if bf16 and any(q[0] >= 16 and q[1] >= 16 for q in qs):
        want[0] = 3
    if not want:
        return -1
    sizes = (_lib.Dim3 * len(qs))(*[_lib.Dim3(1, 256, 256) for _ in qs])
    hq = (_lib.QParams * len(qs))(*[_lib.QParams(a, w, g, 1 if s else 0) for (a, w, g, s) in qs])
    fmt_ids = {(4, 4, -1): 2, (8, 8, -1): 1, (16, 16, -1): 0}
    mine = {fmt_ids[q[:3]] for q in qs if q[:3] in fmt_ids}
    for kid in range(lib.mxmoe_num_kernels()):
        if lib.mxmoe_kernel_policy(kid) != 0:
            continue
        have = {f: v for f, v in kernel_variants(lib, kid).items() if f in mine}
        if have == want and lib.mxmoe_group_gemm_plan(kid, sizes, hq, len(qs), None, None) == 1000 + kid:
            return kid
    raise RuntimeError("quant type not supported")


def gg_permute_inp(hidden: torch.Tensor, topk_ids: torch.Tensor, E: int):
    """ref_bind.cu:47-64 -> (num_problems, inp_buffer [R, K], perm_indices [R], recv_tokens_per_exp [E] int64 CPU)."""
    dst, perm, _slot, recv = build_permutation(topk_ids, E)
    recv_cpu = recv.cpu()
    routed = int(recv_cpu.sum())                            # entries past this were never written (ids out of range are dropped)
    return int((recv_cpu != 0).sum()), hidden.index_select(0, perm[:routed]), perm, recv_cpu


def per_token_prologue(k: int, topk: int) -> bool:
    """Shapes that mxmoe_quant_act_tokens takes: rows of 512 .. 4096 values, a power of two, at most 8 slots per token."""
    return 512 <= k <= 4096 and k & (k - 1) == 0 and 0 < topk <= 8


_LOGIT_DTYPES = {torch.float16: 0, torch.float32: 1, torch.bfloat16: 2}


def route_topk(router_logits: torch.Tensor, topk: int, renormalise: bool = False, out_ids: torch.Tensor | None = None, out_weights: torch.Tensor | None = None):
    """Router logits [T, E] (fp16, fp32 or bf16, on the device) -> (topk_ids int32 [T, k], topk_weights fp32 [T, k]): softmax over the
    experts in fp32, the k largest probabilities in decreasing order (equal ones: lower expert id first), divided by their sum when
    `renormalise` (mxmoe/quant/moe_tracer.py:79-86).  `out_ids` / `out_weights` receive the result when given (no allocation)."""
    lib = _lib.load()
    if router_logits.dtype not in _LOGIT_DTYPES:
        raise ValueError(f"router logits of dtype {router_logits.dtype}: fp16, fp32 or bf16 expected")
    logits = router_logits.contiguous()
    t, e = logits.shape
    dev = logits.device
    ids = out_ids if out_ids is not None else torch.empty((t, topk), dtype=torch.int32, device=dev)
    w = out_weights if out_weights is not None else torch.empty((t, topk), dtype=torch.float32, device=dev)
    assert ids.shape == (t, topk) and ids.dtype == torch.int32 and ids.is_contiguous() and w.shape == (t, topk) and w.dtype == torch.float32 and w.is_contiguous()
    _lib.check(lib, lib.mxmoe_route_topk(logits.data_ptr(), _LOGIT_DTYPES[logits.dtype], t, e, topk, int(bool(renormalise)), ids.data_ptr(), w.data_ptr(), _stream()))
    return ids, w


def build_permutation(topk_ids: torch.Tensor, num_experts: int, with_inverse: bool = False):
    """Stable sort of the flattened expert ids on the device -> (dst_exp_sorted int32 [R], perm_indices int64 [R],
    src_slot int64 [R], recv_tokens_per_exp int64 [E] on the device); with `with_inverse` also row_of_slot int32 [R]: the sorted row
    of every (token, slot), -1 where the expert id was out of range."""
    lib = _lib.load()
    ids = topk_ids.to(torch.int32).contiguous()
    t, k = ids.shape
    r = t * k
    dev = ids.device
    dst = torch.empty(r, dtype=torch.int32, device=dev)
    perm = torch.empty(r, dtype=torch.int64, device=dev)
    slot = torch.empty(r, dtype=torch.int64, device=dev)
    recv = torch.empty(num_experts, dtype=torch.int64, device=dev)
    ws = torch.empty(lib.mxmoe_permute_workspace_bytes(r, num_experts), dtype=torch.uint8, device=dev)
    if with_inverse:
        inv = torch.empty(r, dtype=torch.int32, device=dev)
        _lib.check(lib, lib.mxmoe_build_permutation_inv(ids.data_ptr(), t, k, num_experts, dst.data_ptr(), perm.data_ptr(), slot.data_ptr(), recv.data_ptr(),
                                                        inv.data_ptr(), ws.data_ptr(), _stream()))
        return dst, perm, slot, recv, inv
    _lib.check(lib, lib.mxmoe_build_permutation(ids.data_ptr(), t, k, num_experts, dst.data_ptr(), perm.data_ptr(), slot.data_ptr(), recv.data_ptr(), ws.data_ptr(), _stream()))
    return dst, perm, slot, recv


def _offsets(recv_cpu, num_tokens: int, num_experts: int, has_shared: bool, qparams_per_exp, ld: int, ld_shared: int, bf6: bool = False, fp8: bool = False):
    """Host offset builder of ref_bind.cu:475-505 / 635-671 (units: fp16 elements)."""
    et = num_experts + (1 if has_shared else 0)
    if len(qparams_per_exp) < et:
        raise RuntimeError(f"qparams_per_exp has {len(qparams_per_exp)} entries, need {et}")
    rows, inp_sizes, scale_sizes, lds = [], [], [], []
    cols = [[], [], [], []]                                  # tag, first row, input offset, scale offset per expert
    recv_list = recv_cpu.tolist() if hasattr(recv_cpu, "tolist") else list(recv_cpu)
    acc = io = so = 0
    for e in range(et):
        a_bits, _w, g, _s = qparams_per_exp[e]
        tag = act_tag(int(a_bits), int(g), bf6 and int(_w) == 4, fp8 and int(_w) == 8)
        if tag not in (0, 1, 2, 3, 4, 5):
            raise RuntimeError("quant type not supported")
        width = ld_shared if e == num_experts else ld
        if tag == 3 and width % 128:
            raise RuntimeError(f"group-128 activations need a row length that is a multiple of 128, got {width}")
        if tag == 4 and (width % 128 or width < 256):
            raise RuntimeError(f"bf6 fragments need a row length that is a multiple of 128 and at least 256, got {width}")
        qld = width * 3 // 8 if tag == 4 else (width if tag == 0 else (width // 2 if tag in (1, 5) else width // 4))
        sld = 0 if tag == 0 else (width // 128 if tag == 3 else 1)    # scales per row (ref_bind.cu:492)
        n = num_tokens if e == num_experts else int(recv_list[e])
        for c, v in zip(cols, (tag, acc, io, so)):
            c.append(v)
        rows.append(n)
        inp_sizes.append(packed_elems(tag, n, width))
        scale_sizes.append(sld * n)
        lds.append(qld)
        acc += n
        io += inp_sizes[-1]
        so += sld * n
    return torch.tensor(cols, dtype=torch.int64), rows, inp_sizes, scale_sizes, lds, io, so


def _views(store, scale_store, table, rows, inp_sizes, scale_sizes, lds):
    inp_list, scale_list = [], []
    inp_off, scale_off = table[2].tolist(), table[3].tolist()
    for e, n in enumerate(rows):
        if n == 0:
            continue
        off = inp_off[e]
        inp_list.append(store[off:off + inp_sizes[e]].view(-1, lds[e]))   # [n, row] (tag 4: [32 * blocks, 3/8 of the row]: fragments, not rows)
        soff = scale_off[e]
        scale_list.append(scale_store[soff:soff + scale_sizes[e]])
    return inp_list, scale_list


def quant_inp_act(hidden, topk_ids, num_experts: int, N: int, num_shared_experts: int, qparams_per_exp, verbose: bool = False, rotate: int = 0, bf6: bool = False, fp8: bool = False):
    """ref_bind.cu:434-592.  Returns (inp_list, scale_list, out_list, inp_store, scale_store, out_store,
    recv_tokens_per_exp (int64 CPU), perm_indices, dst_exp_sorted).  The lists are views into the stores, one per
    non-empty problem (shared expert last); out_list[p] is the [M_p, 2N] (shared: [T, 2N * num_shared]) gate_up output buffer."""
    lib = _lib.load()
    assert hidden.dim() == 2 and hidden.dtype == torch.float16 and hidden.is_cuda
    hidden = hidden.contiguous()
    t, k = hidden.shape
    topk = topk_ids.shape[1]
    has_shared = num_shared_experts > 0
    # power-of-two rows without operand variants: quantise a token once per format among its destinations, not once per destination row
    per_token = per_token_prologue(k, topk) and not (bf6 or fp8)
    dst, perm, _slot, recv, *inv = build_permutation(topk_ids, num_experts, with_inverse=per_token)
    recv_cpu = recv.cpu()                                   # one small D2H copy, as ref_bind.cu:451
    table, rows, inp_sizes, scale_sizes, lds, io, so = _offsets(recv_cpu, t, num_experts, has_shared, qparams_per_exp, k, k, bf6, fp8)
    dev = hidden.device
    inp_store = torch.empty(io, dtype=torch.float16, device=dev)
    scale_store = torch.empty(so, dtype=torch.float16, device=dev)
    out_store = torch.empty((num_shared_experts + topk) * t * N * 2, dtype=torch.float16, device=dev)
    d_table = table.to(dev)
    hk, hf, signs = device_signs(k, dev) if rotate else (1, 1, None)
    routed = int(recv_cpu.sum())                            # rows whose expert id was in range; the sorted arrays hold exactly these
    if per_token:
        ids32 = topk_ids.to(torch.int32).contiguous()
        _lib.check(lib, lib.mxmoe_quant_act_tokens(hidden.data_ptr(), inp_store.data_ptr(), scale_store.data_ptr(), ids32.data_ptr(), inv[0].data_ptr(), d_table.data_ptr(),
                                                   k, t, topk, num_experts, int(has_shared), rotate, _stream()))
    else:
        _lib.check(lib, lib.mxmoe_quant_act(hidden.data_ptr(), inp_store.data_ptr(), scale_store.data_ptr(), dst.data_ptr(), perm.data_ptr(), d_table.data_ptr(),
                                            k, routed, t, num_experts, int(has_shared), rotate | (ROWS_VARIANTS if bf6 or fp8 else 0), hk, hf,
                                            None if signs is None else signs.data_ptr(), _stream()))
    inp_list, scale_list = _views(inp_store, scale_store, table, rows, inp_sizes, scale_sizes, lds)
    out_list, off = [], 0
    for e, n in enumerate(rows):
        if n == 0:
            continue
        ld = N * 2 * num_shared_experts if e == num_experts else N * 2
        out_list.append(out_store[off:off + n * ld].view(n, ld))
        off += n * ld
    if verbose:
        for e, n in enumerate(rows):
            print(f"exp: {e} tokens: {n} qinp_size: {inp_sizes[e]} qinp_scale_size: {scale_sizes[e]}")
    return inp_list, scale_list, out_list, inp_store, scale_store, out_store, recv_cpu, perm, dst


def silu_mul_then_quant(inp, num_problems: int, num_experts: int, K: int, N: int, num_shared_experts: int, num_tokens: int, topk: int,
                        values_sorted, recv_tokens_per_exp, qparams_per_exp, rotate: int = 0, bf6: bool = False, fp8: bool = False):
    """ref_bind.cu:595-757.  `inp` is the flat gate_up output store ([R, 2N] routed rows then [T, 2N*num_shared] shared rows),
    `values_sorted` the sorted expert ids.  Returns (inp_list, scale_list, out_list, inp_store, scale_store, out_store) where
    out_list[p] is the [M_p, K] buffer of the down projection."""
    lib = _lib.load()
    has_shared = num_shared_experts > 0
    dev = inp.device
    recv_cpu = recv_tokens_per_exp.cpu()
    r = int(recv_cpu.sum())                                 # routed rows in the store (ids out of range were dropped by the permutation)
    table, rows, inp_sizes, scale_sizes, lds, io, so = _offsets(recv_cpu, num_tokens, num_experts, has_shared, qparams_per_exp, N, N * max(num_shared_experts, 1), bf6, fp8)
    inp_store = torch.empty(io, dtype=torch.float16, device=dev)
    scale_store = torch.empty(so, dtype=torch.float16, device=dev)
    out_store = torch.empty((1 + topk) * num_tokens * K, dtype=torch.float16, device=dev)
    d_table = table.to(dev)
    flat = inp.reshape(-1)
    n_sh = N * num_shared_experts
    hk, hf, signs = device_signs(N, dev) if rotate else (1, 1, None)
    if rotate and has_shared and device_signs(n_sh, dev)[0] != hk:
        raise RuntimeError("routed and shared intermediate sizes need the same Hadamard order")
    shared_ptr = flat.data_ptr() + r * N * 2 * 2
    _lib.check(lib, lib.mxmoe_silu_mul_quant(flat.data_ptr(), shared_ptr, inp_store.data_ptr(), scale_store.data_ptr(), values_sorted.data_ptr(), d_table.data_ptr(),
                                             N, n_sh, r, num_tokens, num_experts, int(has_shared), rotate | (ROWS_VARIANTS if bf6 or fp8 else 0), hk, hf, None if signs is None else signs.data_ptr(), _stream()))
    inp_list, scale_list = _views(inp_store, scale_store, table, rows, inp_sizes, scale_sizes, lds)
    out_list, off = [], 0
    for e, n in enumerate(rows):
        if n == 0:
            continue
        out_list.append(out_store[off:off + n * K].view(n, K))
        off += n * K
    return inp_list, scale_list, out_list, inp_store, scale_store, out_store


def gg_unpermute_out(out_store: torch.Tensor, topk_ids: torch.Tensor, topk_weights: torch.Tensor, num_experts: int, K: int, num_shared_experts: int = 0,
                     output: torch.Tensor | None = None) -> torch.Tensor:
    """The step after the down launch, which the reference leaves as an empty stub (`gg_unpermute_out`, ref_bind.cu:66):
    output[t] = sum_k topk_weights[t, k] * down(row of (t, k)) (+ the shared expert's row t), fp32 accumulation in slot order,
    rounded once to fp16.  `out_store` is the flat down-projection store returned by `silu_mul_then_quant` (routed rows in sorted
    order, then the shared expert's rows)."""
    lib = _lib.load()
    ids = topk_ids.to(torch.int32).contiguous()
    t, k = ids.shape
    w = topk_weights.to(torch.float32).contiguous()
    assert w.shape == (t, k) and w.is_cuda and out_store.is_cuda and out_store.dtype == torch.float16
    _dst, _perm, slot, recv = build_permutation(ids, num_experts)  # stable, so the same order the rows were produced in
    rows = int(recv.sum().item())
    flat = out_store.reshape(-1)
    need = (rows + (t if num_shared_experts else 0)) * K
    if flat.numel() < need:
        raise RuntimeError(f"out_store holds {flat.numel()} elements, the layer produced {need}")
    out = output if output is not None else torch.empty((t, K), dtype=torch.float16, device=flat.device)
    assert out.shape == (t, K) and out.dtype == torch.float16 and out.is_contiguous()
    ws = torch.empty(lib.mxmoe_combine_workspace_bytes(t, k), dtype=torch.uint8, device=flat.device)
    shared_ptr = flat.data_ptr() + rows * K * 2 if num_shared_experts else None
    _lib.check(lib, lib.mxmoe_unpermute_combine(flat.data_ptr(), shared_ptr, w.data_ptr(), slot.data_ptr(), rows, t, k, K, out.data_ptr(), ws.data_ptr(), _stream()))
    return out


def _problem_lists(num_experts: int, experts, recv_cpu, num_tokens: int):
    has_shared = len(experts) > num_experts
    recv_list = recv_cpu.tolist()
    for e in range(num_experts + (1 if has_shared else 0)):
        n = num_tokens if e == num_experts else int(recv_list[e])
        if n:
            yield e, n


def gg_mxmoe_share_fused(inp, experts, scale_zp_a, scale_zp_b, output, N: int, K: int, shared_N: int, shared_K: int, qparams_per_exp,
                         recv_tokens_per_exp, verbose: bool = False, kernel_id: int = -1, acc_dump=None):
    """ref_bind.cu:312-431: one fused launch over every non-empty expert (+ the shared expert as problem index E).

    `inp`, `scale_zp_a`, `output` are indexed by PROBLEM, `experts`, `scale_zp_b`, `qparams_per_exp` by EXPERT
    (ref_bind.cu:362-371).  Returns `output`."""
    plan = prepare_gg(inp, experts, scale_zp_a, scale_zp_b, output, N, K, shared_N, shared_K, qparams_per_exp, recv_tokens_per_exp, kernel_id, acc_dump)
    if verbose:
        print(f"num_problems: {plan.count}")
        for i, (s, q) in enumerate(zip(plan.sizes, plan.qparams)):
            print(f"problem {i}: {list(s)} qparams: {q}")
    plan.run()
    return output


def prepare_gg(inp, experts, scale_zp_a, scale_zp_b, output, N, K, shared_N, shared_K, qparams_per_exp, recv_tokens_per_exp, kernel_id: int = -1, acc_dump=None) -> GroupGemmLaunch:
    """The pointer-table part of `gg_mxmoe_share_fused`, reusable across launches (CUDA-graph friendly)."""
    recv_cpu = recv_tokens_per_exp.cpu()
    e_cnt = recv_cpu.shape[0]
    num_tokens = output[-1].shape[0] if len(output) else 0             # rows of the last problem (the shared expert's, when there is one)
    As, Bs, sa, sb, Cs, sizes, qps = [], [], [], [], [], [], []
    for p, (e, n) in enumerate(_problem_lists(e_cnt, experts, recv_cpu, num_tokens)):
        As.append(inp[p])
        Bs.append(experts[e])
        sa.append(scale_zp_a[p] if scale_zp_a is not None and p < len(scale_zp_a) else None)
        sb.append(scale_zp_b[e] if scale_zp_b is not None else None)
        Cs.append(output[p])
        sizes.append((n, shared_N, shared_K) if e == e_cnt else (n, N, K))
        qps.append(tuple(qparams_per_exp[e]))
    if len(As) != len(inp):
        raise RuntimeError(f"{len(inp)} inputs for {len(As)} non-empty problems")
    g = GroupGemmLaunch(As, Bs, sa, sb, Cs, sizes, qps, kernel_id=kernel_id, acc=acc_dump)
    g.qparams = qps
    return g


def gg_cutlass(inp, experts, topk_ids, output, num_problems=None, inp_buffer=None, perm_indices=None, recv_tokens_per_exp=None):
    """ref_bind.cu:68-182: fp16 grouped GEMM `output[rows of e] = inp[perm rows] @ experts[e].T` (the reference's CUTLASS baseline;
    here the fp16 MFMA branch of the same fused kernel).  experts [E, N, K] fp16, output [T*topk, N]."""
    if inp.dim() != 2:
        raise RuntimeError("hidden must be 2D")
    if not (inp.is_cuda and experts.is_cuda):
        raise RuntimeError("dev must be on cuda")
    e_cnt, n, k = experts.shape
    if perm_indices is None:
        num_problems, inp_buffer, perm_indices, recv_tokens_per_exp = gg_permute_inp(inp, topk_ids, e_cnt)
    recv_cpu = recv_tokens_per_exp.cpu()
    As, Bs, Cs, sizes = [], [], [], []
    st = 0
    for e in range(e_cnt):
        m = int(recv_cpu[e])
        if m == 0:
            continue
        As.append(inp_buffer[st:st + m])
        Bs.append(experts[e])
        Cs.append(output[st:st + m])
        sizes.append((m, n, k))
        st += m
    GroupGemmLaunch(As, Bs, None, None, Cs, sizes, [(16, 16, -1, True)] * len(As)).run()
    return output


def gg_cutlass_share_fused(inp, experts, shared_experts, topk_ids, output, shared_output, num_problems=None, inp_buffer=None, perm_indices=None,
                           recv_tokens_per_exp=None):
    """ref_bind.cu:184-310: as `gg_cutlass` plus one more problem `shared_output = inp @ shared_experts.T` in the same launch."""
    if inp.dim() != 2:
        raise RuntimeError("hidden must be 2D")
    if not (inp.is_cuda and experts.is_cuda):
        raise RuntimeError("dev must be on cuda")
    e_cnt, n, k = experts.shape
    n_sh, k_sh = shared_experts.shape
    if perm_indices is None:
        num_problems, inp_buffer, perm_indices, recv_tokens_per_exp = gg_permute_inp(inp, topk_ids, e_cnt)
    recv_cpu = recv_tokens_per_exp.cpu()
    As, Bs, Cs, sizes = [], [], [], []
    st = 0
    for e in range(e_cnt):
        m = int(recv_cpu[e])
        if m == 0:
            continue
        As.append(inp_buffer[st:st + m])
        Bs.append(experts[e])
        Cs.append(output[st:st + m])
        sizes.append((m, n, k))
        st += m
    As.append(inp)
    Bs.append(shared_experts)
    Cs.append(shared_output)
    sizes.append((inp.shape[0], n_sh, k_sh))
    GroupGemmLaunch(As, Bs, None, None, Cs, sizes, [(16, 16, -1, True)] * len(As)).run()
    return output
