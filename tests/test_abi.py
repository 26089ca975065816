"""CPU checks of the C-ABI boundary: the library loads, exports every symbol the header declares, and its host-only
entry points (registry, launch planning, error paths) behave.  No kernel is launched here."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_header_symbols_are_exported_and_bound(lib):
    from mxmoe_amd import _lib

    header = (ROOT / "include" / "mxmoe_amd.h").read_text()
    declared = set(re.findall(r"\b(mxmoe_[a-z0-9_]+)\s*\(", header))
    declared -= {"mxmoe_dim3", "mxmoe_qparams"}
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/mxmoe_amd.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert set(_lib.SIGNATURES) == declared


def test_struct_layouts_match_the_reference_sizes():
    from mxmoe_amd import _lib

    assert C.sizeof(_lib.QParams) == 16 and C.sizeof(_lib.Dim3) == 12      # QParams quantize.cuh:14-25, dim3


def test_registry_names_follow_the_reference_format(lib):
    n = lib.mxmoe_num_kernels()
    assert n >= 4
    names = [lib.mxmoe_kernel_name(i).decode() for i in range(n)]
    assert any(re.match(r"\[w4a4_g-1_sym: \(\d+,\d+,\d+\) \(\d,\d,1\) \d\], ", s) for s in names)
    assert lib.mxmoe_find_kernel(b"groupgemm_hz_fused_wxax") == 0
    assert lib.mxmoe_find_kernel(b"nope") == -1
    out = (C.c_int32 * 8)()
    assert lib.mxmoe_kernel_branch(0, 0, out) == 0 and out[1] % 32 == 0 and out[2] % 64 == 0
    assert lib.mxmoe_kernel_branch(0, 99, out) != 0 and b"branch" in lib.mxmoe_last_error()


def _plan(lib, kernel, probs):
    from mxmoe_amd import _lib

    sizes = (_lib.Dim3 * len(probs))(*[_lib.Dim3(*p[0]) for p in probs])
    qs = (_lib.QParams * len(probs))(*[_lib.QParams(p[1][0], p[1][1], p[1][2], int(p[1][3])) for p in probs])
    br = (C.c_int32 * len(probs))()
    tiles = C.c_int32()
    rc = lib.mxmoe_group_gemm_plan(kernel, sizes, qs, len(probs), br, C.byref(tiles))
    return rc, list(br), tiles.value


def test_plan_counts_tiles_like_the_reference_launcher(lib):
    # kernel_sketch.py:89-101: total += cdiv(M, BM) * cdiv(N, BN) per problem with the tile of its qcfg
    probs = [((546, 2816, 2048), (4, 4, -1, True)), ((0, 2816, 2048), (8, 8, -1, True)), ((20, 2048, 1408), (8, 8, -1, True))]
    rc, br, tiles = _plan(lib, -1, probs)
    assert rc == 1000                                                     # first registered kernel covers w4a4 + w8a8
    out = (C.c_int32 * 8)()
    # 546 rows of w4a4 run as two segments: 4 whole 128 x 256 tile rows, then the 34 remaining rows with one 64 x 256 tile row
    lib.mxmoe_kernel_branch(0, br[0], out)
    assert (out[1], out[2]) == (128, 256)
    exp = 4 * (2816 // 256) + 1 * (2816 // 256) + 0 + 1 * (2048 // 256)
    assert tiles == exp
    lib.mxmoe_kernel_branch(0, br[2], out)
    assert out[0] == 1 and out[1] == 32                                  # 20 rows of w8a8 -> the 32-row w8a8 tile


def test_unsupported_format_message(lib):
    rc, _, _ = _plan(lib, -1, [((8, 256, 128), (8, 4, -1, True))])
    assert rc == 1 and lib.mxmoe_last_error() == b"quant type not supported"   # compose_kernel.py:433
    rc, _, _ = _plan(lib, -1, [((8, 256, 128), (16, 4, 128, False)), ((8, 256, 128), (4, 4, -1, True)), ((8, 256, 128), (16, 16, -1, True))])
    assert rc >= 1000 and b"fused_all" in lib.mxmoe_kernel_name(rc - 1000)


def test_missing_library_fails_loudly(tmp_path):
    from mxmoe_amd import _lib

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load(tmp_path / "libmissing.so")


def test_plan_bounds_on_random_problem_lists(lib):
    """Host planner on random problem lists (every format, empty problems, lists longer than one launch's table): it never fails, and
    the tile count lies between what the largest and the smallest tile shapes of the chosen kernel would need."""
    import random

    rnd = random.Random(7)
    fmts = [((4, 4, -1, True), 128), ((8, 8, -1, True), 64), ((16, 4, 128, False), 128), ((16, 3, 128, False), 128), ((16, 2, 128, True), 128),
            ((16, 16, -1, True), 32), ((4, 4, 128, True), 128)]
    out = (C.c_int32 * 8)()
    for trial in range(40):
        nprob = rnd.choice([1, 3, 17, 60, 121, 260])
        pick = rnd.sample(fmts, rnd.choice([1, 2, 3]))
        probs = []
        for _ in range(nprob):
            q, kmul = rnd.choice(pick)
            m = rnd.choice([0, 1, 7, 31, 32, 33, 100, 129, 546, 5000, 40000])
            n = 16 * rnd.randint(1, 400)
            k = kmul * rnd.randint(1, 40)
            probs.append(((m, n, k), q))
        rc, br, tiles = _plan(lib, -1, probs)
        assert rc >= 1000, (lib.mxmoe_last_error(), probs[:3])
        kid = rc - 1000
        shapes = []
        for b in range(lib.mxmoe_kernel_num_branches(kid)):
            assert lib.mxmoe_kernel_branch(kid, b, out) == 0
            shapes.append((out[0], out[1], out[2]))
        lo = hi = 0
        fmt_id = {(4, 4, -1): 2, (8, 8, -1): 1, (16, 4, 128): 3, (16, 3, 128): 4, (16, 2, 128): 5, (16, 16, -1): 0, (4, 4, 128): 6}
        for (m, n, k), q in probs:
            mine = [(bm, bn) for f, bm, bn in shapes if f == fmt_id[(q[0], q[1], q[2])]]
            assert mine, "the chosen kernel has a tile for every format of the list"
            if m == 0:
                continue
            lo += min(-(-m // bm) * -(-n // bn) for bm, bn in mine if bm == max(x for x, _ in mine))
            hi += max(-(-m // bm) * -(-n // bn) for bm, bn in mine)
        assert lo <= tiles <= hi, (trial, lo, tiles, hi)


def test_missing_arrays_are_refused_before_any_launch(lib):
    """A quantised problem without scale arrays, or a plan without its host arrays, fails on the host with code 5."""
    from mxmoe_amd import _lib

    sizes = (_lib.Dim3 * 1)(_lib.Dim3(8, 256, 128))
    q = (_lib.QParams * 1)(_lib.QParams(4, 4, -1, 1))
    one = (C.c_void_p * 1)(0)
    addr = C.addressof(one)
    rc = lib.mxmoe_group_gemm(0, addr, addr, None, None, addr, addr, None, None, None, None, addr, sizes, None, q, 1, None, None)
    assert rc == 5 and b"scale arrays" in lib.mxmoe_last_error()
    rc = lib.mxmoe_group_gemm(0, None, addr, addr, addr, addr, addr, None, None, None, None, addr, sizes, None, q, 1, None, None)
    assert rc == 5 and b"null argument" in lib.mxmoe_last_error()
    assert lib.mxmoe_group_gemm_plan(-1, None, None, 1, None, None) == 5


def test_ds_is_accepted_and_ignored(lib):
    """The reference's caller hands the kernels a second pointer array Ds with the same entries as Cs (test.cu:446-459) and its
    kernels store through Cs only (hz_fused.cuh:89,110): a distinct Ds array is no error here either.  Host-only: the call
    below passes every check up to the launch and is refused for its (missing) scale arrays, not for its Ds."""
    from mxmoe_amd import _lib

    sizes = (_lib.Dim3 * 1)(_lib.Dim3(8, 256, 128))
    q = (_lib.QParams * 1)(_lib.QParams(4, 4, -1, 1))
    one, other = (C.c_void_p * 1)(0), (C.c_void_p * 1)(0)
    a, b = C.addressof(one), C.addressof(other)
    rc = lib.mxmoe_group_gemm(0, a, a, None, None, a, b, None, None, None, None, a, sizes, None, q, 1, None, None)
    assert rc == 5 and b"scale arrays" in lib.mxmoe_last_error()
    empty = (_lib.Dim3 * 1)(_lib.Dim3(0, 256, 128))                       # no rows: nothing to launch, every check passed
    assert lib.mxmoe_group_gemm(0, a, a, a, a, a, b, None, None, None, None, a, empty, None, q, 1, None, None) == 0


def test_every_tile_is_run_by_exactly_one_workgroup_of_an_oversized_grid(lib):
    """A planned launch is enqueued with a grid sized for the worst routing.  The function the kernels call to find their tile,
    evaluated on the host over such a grid: every tile of the launch exactly once, every surplus workgroup without a tile
    (a surplus workgroup folded back into the last phase would run one of its tiles a second time)."""
    import random

    from mxmoe_amd import _lib

    rnd = random.Random(5)
    fmts = [((4, 4, -1, True), 128), ((8, 8, -1, True), 64), ((16, 4, 128, False), 128), ((16, 16, -1, True), 32)]
    for trial in range(30):
        pick = rnd.sample(fmts, rnd.choice([1, 2, 3]))
        probs = []
        for _ in range(rnd.choice([1, 5, 60, 120])):
            q, kmul = rnd.choice(pick)
            probs.append(((rnd.choice([0, 1, 31, 33, 100, 129, 546, 3000]), 16 * rnd.randint(1, 200), kmul * rnd.randint(1, 20)), q))
        if trial == 0:
            probs = [((0, 256, 128), (4, 4, -1, True))] * 3                # a launch without any tile
        rc, _, tiles = _plan(lib, -1, probs)
        assert rc >= 1000
        sizes = (_lib.Dim3 * len(probs))(*[_lib.Dim3(*p[0]) for p in probs])
        qs = (_lib.QParams * len(probs))(*[_lib.QParams(p[1][0], p[1][1], p[1][2], int(p[1][3])) for p in probs])
        grid = tiles + 8 * 9 + rnd.choice([0, 8, 200, 1000])
        out = (C.c_int32 * grid)()
        assert lib.mxmoe_group_gemm_plan_tile_map(rc - 1000, sizes, qs, len(probs), grid, out) == 0, lib.mxmoe_last_error()
        seen = sorted(t for t in out if t >= 0)
        assert seen == list(range(tiles)), (trial, tiles, len(seen))


def test_kernels_are_exported_with_the_reference_function_type(lib):
    """One function of the reference's FuncType per kernel, by index and by name; a failing call reports through
    mxmoe_last_status (the type returns void).  Host-only: the call below fails validation before any launch."""
    from mxmoe_amd import _lib

    n = lib.mxmoe_num_kernels()
    funcs = [lib.mxmoe_kernel_func(i) for i in range(n)]
    assert all(funcs) and len(set(funcs)) == n                              # every kernel its own function
    assert lib.mxmoe_kernel_func(n) is None and lib.mxmoe_get_kernel(b"nope") is None
    assert lib.mxmoe_get_kernel(b"groupgemm_hz_fused_wxax") == funcs[0]
    assert lib.mxmoe_get_kernel(lib.mxmoe_kernel_name(2)) == funcs[2]       # the full registry key works as well
    assert {lib.mxmoe_kernel_policy(i) for i in range(n)} == {0, 1, 2} and lib.mxmoe_kernel_policy(-1) == -1
    assert lib.mxmoe_get_stream() is None
    lib.mxmoe_set_stream(0x10)
    assert lib.mxmoe_get_stream() == 0x10
    lib.mxmoe_set_stream(None)
    fn = _lib.FUNC_TYPE(funcs[1])                                           # the fp16 kernel, asked to run a w4a4 problem
    sizes = (_lib.Dim3 * 1)(_lib.Dim3(8, 256, 128))
    q = (_lib.QParams * 1)(_lib.QParams(4, 4, -1, 1))
    one = (C.c_void_p * 1)(0)
    a = C.addressof(one)
    fn(a, a, a, a, a, a, None, None, None, None, a, sizes, None, q, 1)
    assert lib.mxmoe_last_status() == 1 and lib.mxmoe_last_error() == b"quant type not supported"
    fn(a, a, a, a, a, a, None, None, None, None, a, sizes, None, q, 0)      # an empty problem list is a successful no-op
    assert lib.mxmoe_last_status() == 0


def test_prologue_entry_points_validate_on_the_host(lib):
    one = (C.c_int64 * 8)()
    a = C.addressof(one)
    assert lib.mxmoe_quant_act(None, a, a, a, a, a, 256, 4, 2, 2, 0, 0, 1, 1, None, None) == 5 and b"null" in lib.mxmoe_last_error()
    assert lib.mxmoe_quant_act(a, a, a, None, a, a, 256, 4, 2, 2, 0, 0, 1, 1, None, None) == 5
    assert lib.mxmoe_quant_act(a, a, a, a, a, a, 256, -1, 2, 2, 0, 0, 1, 1, None, None) == 3
    assert lib.mxmoe_quant_act(a, a, a, a, a, a, 260, 4, 2, 2, 0, 0, 1, 1, None, None) == 3 and b"multiple of 8" in lib.mxmoe_last_error()
    assert lib.mxmoe_silu_mul_quant(a, None, a, a, a, a, 256, 256, 4, 2, 2, 1, 0, 1, 1, None, None) == 5
    assert lib.mxmoe_quant_act_tokens(None, a, a, a, a, a, 2048, 4, 2, 2, 0, 0, None) == 5 and b"null" in lib.mxmoe_last_error()
    assert lib.mxmoe_quant_act_tokens(a, a, a, a, a, a, 1408, 4, 2, 2, 0, 0, None) == 3 and b"512" in lib.mxmoe_last_error()
    assert lib.mxmoe_quant_act_tokens(a, a, a, a, a, a, 2048, 4, 9, 2, 0, 0, None) == 3 and b"8 slots" in lib.mxmoe_last_error()
    assert lib.mxmoe_quant_act_tokens(a, a, a, a, a, a, 2048, 4, 2, 2, 0, 4, None) == 3
    assert lib.mxmoe_quant_act_tokens(a, a, a, a, a, a, 2048, 0, 2, 2, 0, 0, None) == 0      # no tokens: nothing to launch
    assert lib.mxmoe_silu_mul_quant(a, a, a, a, a, a, 1408, 1408, 4, 2, 2, 0, 1, 176, 4, None, None) == 3 and b"sign table" in lib.mxmoe_last_error()
    assert lib.mxmoe_permute_plan_layer(a, 200, 2, 8, a, a, a, a, a, a, a, 0, None) == 3 and b"256" in lib.mxmoe_last_error()   # larger batches: the two separate calls
    assert lib.mxmoe_permute_plan_layer(a, 4, 2, 8, a, a, a, a, a, None, a, 0, None) == 5
    assert lib.mxmoe_permute_plan_layer_ws(a, 100000, 8, 256, a, a, a, a, a, a, a, 0, a, None) == 3 and b"16384" in lib.mxmoe_last_error()
    assert lib.mxmoe_permute_plan_layer_ws(a, 2000, 2, 8, a, a, a, a, a, a, a, 0, None, None) == 5             # no workspace
    assert lib.mxmoe_build_permutation(None, 4, 2, 8, a, a, a, a, a, None) == 5
    assert lib.mxmoe_route_topk(a, 1, 4, 8, 9, 0, a, a, None) == 3 and b"top-k" in lib.mxmoe_last_error()      # k > experts
    assert lib.mxmoe_route_topk(a, 1, 4, 5000, 2, 0, a, a, None) == 3
    assert lib.mxmoe_route_topk(a, 3, 4, 8, 2, 0, a, a, None) == 3                                              # unknown dtype
    assert lib.mxmoe_route_topk(a, 1, 4, 8, 2, 0, None, a, None) == 5
    assert lib.mxmoe_route_topk(None, 1, 0, 8, 2, 0, None, None, None) == 0                                     # no tokens: nothing to launch
    assert lib.mxmoe_build_permutation(a, 0, 2, 8, a, a, a, a, a, None) == 3


def test_planned_grid_bound_covers_every_routing(lib):
    """The worst-case grid of a planned launch against the tile count the host launcher plans for random routings of the same
    total: the bound must never be smaller (a smaller grid would silently drop tiles), and stays within a small factor."""
    import random

    from mxmoe_amd import _lib

    rnd = random.Random(11)
    cases = [([(4, 4, -1, True), (8, 8, -1, True)], 2816, 2048, 60, 32768, 0), ([(16, 4, 128, False), (16, 3, 128, False)], 2816, 2048, 64, 192, 32),
             ([(4, 4, -1, True), (8, 8, -1, True), (16, 4, 128, False)], 28672, 4096, 8, 16384, 0), ([(16, 16, -1, True)], 2816, 2048, 60, 2048, 0),
             ([(4, 4, 128, True), (4, 4, -1, True)], 2048, 1408, 17, 999, 7)]
    for fmts, n, k, e_cnt, routed, shared_rows in cases:
        et = e_cnt + (1 if shared_rows else 0)
        qs = [rnd.choice(fmts) for _ in range(et)]
        desc = (_lib.BlockDesc * et)(*[_lib.BlockDesc(q[0], q[1], q[2], int(q[3]), (C.c_uint8 * 3)(), n, k, 0, 0) for q in qs])
        kid = lib.mxmoe_plan_select_kernel(-1, desc, et)
        assert kid >= 0, lib.mxmoe_last_error()
        bound = lib.mxmoe_plan_grid_bound(kid, desc, e_cnt, routed, shared_rows)
        assert bound > 0, lib.mxmoe_last_error()
        worst = 0
        for trial in range(60):
            style = trial % 4
            if style == 0:                                          # everything on one expert
                counts = [0] * e_cnt
                counts[rnd.randrange(e_cnt)] = routed
            elif style == 1:                                        # as even as possible
                counts = [routed // e_cnt + (1 if i < routed % e_cnt else 0) for i in range(e_cnt)]
            elif style == 2:                                        # many experts just past a tile boundary
                unit = rnd.choice([1, 17, 33, 65, 129])
                counts = [0] * e_cnt
                left = routed
                for i in range(e_cnt):
                    take = min(left, unit)
                    counts[i] = take
                    left -= take
                counts[0] += left
            else:
                cuts = sorted(rnd.randint(0, routed) for _ in range(e_cnt - 1))
                counts = [b - a for a, b in zip([0] + cuts, cuts + [routed])]
            assert sum(counts) == routed
            rows = counts + ([shared_rows] if shared_rows else [])
            rc, _, tiles = _plan(lib, kid, [((m, n, k), q) for m, q in zip(rows, qs)])
            assert rc == 1000 + kid
            worst = max(worst, tiles)
            assert tiles + 8 * 9 <= bound, (fmts, counts[:6], tiles, bound)   # + the padding of every phase to the XCD count
        assert bound <= 2.5 * worst + 600, (fmts, worst, bound)
    bad = (_lib.BlockDesc * 1)(_lib.BlockDesc(8, 4, -1, 1, (C.c_uint8 * 3)(), 256, 128, 0, 0))
    assert lib.mxmoe_plan_select_kernel(-1, bad, 1) < 0 and lib.mxmoe_last_error() == b"quant type not supported"
    assert lib.mxmoe_plan_select_kernel(-1, desc, 4097) < 0               # checked before any entry is read
    assert lib.mxmoe_plan_bytes(130) >= 2 * 4096 + 130 * (32 + 40 + 12)   # a block of more than 120 experts: one table header per launch
    assert lib.mxmoe_plan_bytes(60) >= 4096 + 60 * (32 + 40 + 12)
