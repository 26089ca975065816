"""ctypes loader of libmxmoe_amd.so.  There is no CPU fallback: a missing library is an error."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libmxmoe_amd.so"


class Dim3(C.Structure):
    _fields_ = [("x", C.c_uint32), ("y", C.c_uint32), ("z", C.c_uint32)]


class PlanCall(C.Structure):
    """mxmoe_plan_call."""
    _fields_ = [("kernel_id", C.c_int), ("d_desc", C.c_void_p), ("h_desc", C.c_void_p), ("inp_store", C.c_void_p), ("scale_store", C.c_void_p),
                ("out_store", C.c_void_p), ("d_plan", C.c_void_p)]


class BlockDesc(C.Structure):
    """mxmoe_block_desc: one linear block of one expert for the device-side planner (40 bytes)."""
    _fields_ = [("a_bits", C.c_int32), ("w_bits", C.c_int32), ("gsize", C.c_int32), ("sym", C.c_uint8), ("_pad", C.c_uint8 * 3),
                ("N", C.c_uint32), ("K", C.c_uint32), ("B", C.c_void_p), ("scale_b", C.c_void_p)]


class QParams(C.Structure):
    _fields_ = [("a_bits", C.c_int32), ("w_bits", C.c_int32), ("gsize", C.c_int32), ("sym", C.c_uint8), ("_pad", C.c_uint8 * 3)]


_P = C.c_void_p
_I = C.c_int

# name -> (restype, argtypes); mirrors include/mxmoe_amd.h declaration by declaration
SIGNATURES = {
    "mxmoe_last_error": (C.c_char_p, []),
    "mxmoe_num_kernels": (_I, []),
    "mxmoe_kernel_name": (C.c_char_p, [_I]),
    "mxmoe_find_kernel": (_I, [C.c_char_p]),
    "mxmoe_kernel_num_branches": (_I, [_I]),
    "mxmoe_kernel_branch": (_I, [_I, _I, C.POINTER(C.c_int32)]),
    "mxmoe_group_gemm": (_I, [_I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, C.POINTER(Dim3), _P, C.POINTER(QParams), _I, _P, _P]),
    "mxmoe_permute_workspace_bytes": (C.c_size_t, [_I, _I]),
    "mxmoe_build_permutation": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "mxmoe_route_topk": (_I, [_P, _I, _I, _I, _I, _I, _P, _P, _P]),
    "mxmoe_build_permutation_inv": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P]),
    "mxmoe_combine_planned": (_I, [_P, _P, _I, _P, _P, _I, _I, _I, _P, _P]),
    "mxmoe_static_scratch_bytes": (C.c_size_t, []),
    "mxmoe_build_permutation_static": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P]),
    "mxmoe_quant_act": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
    "mxmoe_quant_act_tokens": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "mxmoe_silu_mul_quant": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
    "mxmoe_group_gemm_plan": (_I, [_I, C.POINTER(Dim3), C.POINTER(QParams), _I, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "mxmoe_kernel_func": (_P, [_I]),
    "mxmoe_get_kernel": (_P, [C.c_char_p]),
    "mxmoe_kernel_policy": (_I, [_I]),
    "mxmoe_set_stream": (None, [_P]),
    "mxmoe_get_stream": (_P, []),
    "mxmoe_last_status": (_I, []),
    "mxmoe_plan_bytes": (C.c_size_t, [_I]),
    "mxmoe_plan_offset": (C.c_size_t, [_I, _I]),
    "mxmoe_plan_select_kernel": (_I, [_I, _P, _I]),
    "mxmoe_plan_grid_bound": (_I, [_I, _P, _I, _I, _I]),
    "mxmoe_plan_block": (_I, [_I, _P, _I, _I, _P, _P, _P, _P, _P, _P, _P]),
    "mxmoe_plan_layer": (_I, [_P, _P, _P, _I, _I, _P]),
    "mxmoe_permute_plan_layer": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P]),
    "mxmoe_permute_plan_layer_ws": (_I, [_P, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _I, _P, _P]),
    "mxmoe_group_gemm_planned": (_I, [_I, _P, _I, _I, _P]),
    "mxmoe_quant_act_planned": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
    "mxmoe_silu_mul_quant_planned": (_I, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _P, _P]),
    "mxmoe_unpermute_combine_planned": (_I, [_P, _P, _I, _P, _P, _I, _I, _I, _P, _P, _P]),
    "mxmoe_group_gemm_plan_tables": (_I, [_I, C.POINTER(Dim3), C.POINTER(QParams), _I, C.POINTER(C.c_int32), _I]),
    "mxmoe_group_gemm_plan_tile_map": (_I, [_I, C.POINTER(Dim3), C.POINTER(QParams), _I, _I, C.POINTER(C.c_int32)]),
    "mxmoe_combine_workspace_bytes": (C.c_size_t, [_I, _I]),
    "mxmoe_unpermute_combine": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _P, _P, _P]),
}

_cached = {}


GEMM_ONLY = ("mxmoe_last_error", "mxmoe_num_kernels", "mxmoe_kernel_name", "mxmoe_find_kernel", "mxmoe_kernel_num_branches", "mxmoe_kernel_branch",
             "mxmoe_group_gemm", "mxmoe_group_gemm_plan", "mxmoe_group_gemm_plan_tables", "mxmoe_group_gemm_plan_tile_map", "mxmoe_kernel_func", "mxmoe_get_kernel", "mxmoe_kernel_policy", "mxmoe_set_stream", "mxmoe_get_stream",
             "mxmoe_last_status")

# the reference's FuncType (registry.cuh:28-39): 15 arguments, no return value
FUNC_TYPE = C.CFUNCTYPE(None, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, C.POINTER(Dim3), _P, C.POINTER(QParams), _I)


def load(path: str | Path | None = None) -> C.CDLL:
    """Load the library and attach the C-ABI signatures.  A generated library (`path` given) carries the GroupGEMM entry
    points only; the default library must export everything the header declares."""
    p = Path(path) if path is not None else LIB_PATH
    hit = _cached.get(str(p))  # (as given: the operators come here on every call and should not walk the file system again)
    if hit is not None:
        return hit
    if not p.exists():
        raise RuntimeError(
            f"{p} is missing: build it with `python -m mxmoe_amd.build` (hipcc, gfx950). "
            "mxmoe_amd has no CPU fallback for its kernels."
        )
    # one handle per file name: the system loader caches shared libraries by name too (generated libraries carry a digest of
    # their kernel set in their name, so a different set is a different file)
    key = str(p.resolve())
    if key in _cached:
        return _cached[key]
    lib = C.CDLL(str(p))
    for name, (res, args) in SIGNATURES.items():
        if path is not None and name not in GEMM_ONLY and not hasattr(lib, name):
            continue
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _cached[key] = _cached[str(p)] = lib
    return lib


def check(lib: C.CDLL, rc: int) -> None:
    if rc != 0:
        raise RuntimeError(lib.mxmoe_last_error().decode())
