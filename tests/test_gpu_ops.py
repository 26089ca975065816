"""GPU tests of the operator names a caller of the reference's `mxmoe_ops` module uses besides the fused mixed-precision path:
`gg_permute_inp`, `gg_cutlass`, `gg_cutlass_share_fused` (mxmoe/kernels/src/ref_bind.cu:47-64, 68-182, 184-310), of a kernel
library produced by the template generator, and of the sequential / multi-stream launch policies."""
import numpy as np
import pytest
import torch

from oracle import mxmoe_oracle as O

pytestmark = pytest.mark.gpu
F16 = np.float16
DEV = "cuda"


def _rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return np.abs(a - b).max() / max(np.abs(b).max(), 1e-6)


def _routing(rng, t, e, k, leave_empty=()):
    logits = rng.standard_normal((t, e)).astype(np.float32)
    logits[:, list(leave_empty)] = -1e9
    ids, _ = O.route_topk(logits, k)
    return ids


def test_gg_permute_inp_matches_the_stable_permutation():
    from mxmoe_amd import ops

    rng = np.random.default_rng(3)
    t, e, k, hid = 97, 12, 3, 64
    ids = _routing(rng, t, e, k, leave_empty=(4, 11))
    hidden = rng.standard_normal((t, hid)).astype(F16)
    n_prob, buf, perm, recv = ops.gg_permute_inp(torch.from_numpy(hidden).to(DEV), torch.from_numpy(ids).to(DEV), e)
    _, o_perm, _, o_recv = O.permute_by_expert(ids, e)
    assert n_prob == int((o_recv > 0).sum()) == e - 2
    assert not recv.is_cuda and np.array_equal(recv.numpy(), o_recv)            # int64 on the host, as ref_bind.cu:59-61
    assert np.array_equal(perm.cpu().numpy(), o_perm)
    assert np.array_equal(buf.cpu().numpy().view(np.uint16), hidden[o_perm].view(np.uint16))


@pytest.mark.parametrize("reuse_permutation", [False, True])
def test_gg_cutlass_fp16_grouped_gemm(reuse_permutation):
    """output[rows of e] = hidden[perm rows] @ experts[e].T against the oracle's fp16 GEMM (fp64 accumulation, one rounding) to
    max-abs-rel 1e-2; experts without tokens contribute no problem."""
    from mxmoe_amd import ops

    rng = np.random.default_rng(4)
    t, e, k, hid, n = 150, 6, 2, 256, 384
    ids = _routing(rng, t, e, k, leave_empty=(2,))
    hidden = rng.standard_normal((t, hid)).astype(F16)
    experts = (rng.standard_normal((e, n, hid)) * 0.05).astype(F16)
    d_h, d_e, d_ids = (torch.from_numpy(a).to(DEV) for a in (hidden, experts, ids))
    out = torch.full((t * k, n), float("nan"), dtype=torch.float16, device=DEV)
    extra = ops.gg_permute_inp(d_h, d_ids, e) if reuse_permutation else ()
    res = ops.gg_cutlass(d_h, d_e, d_ids, out, *extra)
    torch.cuda.synchronize()
    assert res is out
    _, perm, _, recv = O.permute_by_expert(ids, e)
    got, st = out.cpu().numpy(), 0
    for ex in range(e):
        m = int(recv[ex])
        want = O.gemm_fp16(hidden[perm[st:st + m]], experts[ex])
        assert m == 0 or _rel(got[st:st + m], want) <= 1e-2, f"expert {ex}"
        st += m
    assert st == t * k and np.isfinite(got).all()


def test_gg_cutlass_share_fused_adds_the_shared_problem():
    from mxmoe_amd import ops

    rng = np.random.default_rng(5)
    t, e, k, hid, n, n_sh = 40, 5, 2, 128, 256, 512
    ids = _routing(rng, t, e, k)
    hidden = rng.standard_normal((t, hid)).astype(F16)
    experts = (rng.standard_normal((e, n, hid)) * 0.05).astype(F16)
    shared = (rng.standard_normal((n_sh, hid)) * 0.05).astype(F16)
    d_h, d_e, d_s, d_ids = (torch.from_numpy(a).to(DEV) for a in (hidden, experts, shared, ids))
    out = torch.full((t * k, n), float("nan"), dtype=torch.float16, device=DEV)
    out_sh = torch.full((t, n_sh), float("nan"), dtype=torch.float16, device=DEV)
    ops.gg_cutlass_share_fused(d_h, d_e, d_s, d_ids, out, out_sh)
    torch.cuda.synchronize()
    _, perm, _, recv = O.permute_by_expert(ids, e)
    got, st = out.cpu().numpy(), 0
    for ex in range(e):
        m = int(recv[ex])
        assert m == 0 or _rel(got[st:st + m], O.gemm_fp16(hidden[perm[st:st + m]], experts[ex])) <= 1e-2, f"expert {ex}"
        st += m
    assert _rel(out_sh.cpu().numpy(), O.gemm_fp16(hidden, shared)) <= 1e-2


def test_gg_cutlass_argument_checks():
    from mxmoe_amd import ops

    with pytest.raises(RuntimeError, match="2D"):
        ops.gg_cutlass(torch.zeros(2, 3, 4, dtype=torch.float16, device=DEV), torch.zeros(1, 8, 4, dtype=torch.float16, device=DEV),
                       torch.zeros(2, 1, dtype=torch.int32, device=DEV), torch.zeros(2, 8, dtype=torch.float16, device=DEV))
    with pytest.raises(RuntimeError, match="cuda"):
        ops.gg_cutlass(torch.zeros(2, 4, dtype=torch.float16), torch.zeros(1, 8, 4, dtype=torch.float16),
                       torch.zeros(2, 1, dtype=torch.int32), torch.zeros(2, 8, dtype=torch.float16))


def _mixed_problems(rng):
    from test_gpu_group_gemm import _wxax_problem

    shapes = [(1, 256, 128, 4), (31, 512, 256, 8), (33, 384, 1408, 4), (130, 256, 256, 8), (300, 768, 384, 4), (64, 2816, 2048, 4),
              (129, 2048, 1408, 8), (17, 264, 128, 8), (520, 512, 512, 8), (5, 256, 2048, 4)]
    return [_wxax_problem(rng, m, n, k, b) for (m, n, k, b) in shapes]


def test_generated_library_mixed_launch_is_bit_exact():
    """The reference's flow generator -> build -> registry -> launch (mxmoe/kernels/compose_kernel.py:532-572,
    run_mxmoe_gg.py:99-121): the library the template generator emitted for {w4a4, w8a8} (one-tile-per-format combinations and a
    kernel of shape sets; compiled by the package build) is loaded through the product's loader and every kernel it registers runs
    one mixed launch whose accumulators and outputs equal the oracle's bit for bit."""
    from mxmoe_amd import _lib, build
    from mxmoe_amd.group_gemm import GroupGemmLaunch

    gen = build.sample_generator()
    gen.kernel_names = [f"groupgemm_{gen.kernel_type}_{i}" for i in range(len(gen.get_tile_configs()))]
    lib = _lib.load(gen.library_path())                                      # raises when the build did not produce it
    assert lib.mxmoe_num_kernels() == len(gen.kernel_names) == 5
    probs = _mixed_problems(np.random.default_rng(21))
    for kid in range(lib.mxmoe_num_kernels()):
        name = lib.mxmoe_kernel_name(kid).decode()
        assert name.endswith(gen.kernel_names[kid]) and "w4a4_g-1_sym" in name and "w8a8_g-1_sym" in name
        Cs = [torch.full(p["size"][:2], float("nan"), dtype=torch.float16, device=DEV) for p in probs]
        accs = [torch.zeros(p["size"][:2], dtype=torch.int32, device=DEV) for p in probs]
        g = GroupGemmLaunch([p["A"] for p in probs], [p["B"] for p in probs], [p["sa"] for p in probs], [p["sb"] for p in probs], Cs,
                            [p["size"] for p in probs], [p["q"] for p in probs], kernel_id=kid, acc=accs, lib=lib)
        g.run()
        torch.cuda.synchronize()
        for p, c, a in zip(probs, Cs, accs):
            assert np.array_equal(a.cpu().numpy(), p["acc"]), f"{name}: accumulators of {p['size']} {p['q']}"
            assert np.array_equal(c.cpu().numpy().view(np.uint16), p["out"].view(np.uint16)), f"{name}: outputs of {p['size']} {p['q']}"


def test_sequential_and_multistream_policies_give_the_fused_bits():
    """The ablation launchers of the reference (one launch per run of equal-format problems, on one stream or on one stream per
    run: mxmoe/kernels/kernel_sketch.py:148-274, 277-406) compute what the one fused launch computes."""
    from mxmoe_amd import harness

    probs = _mixed_problems(np.random.default_rng(22))
    for p in probs:
        p["C"] = torch.full(p["size"][:2], float("nan"), dtype=torch.float16, device=DEV)
    lib = None
    fused = harness.launch_policy(probs, "fused", lib)
    fused()
    torch.cuda.synchronize()
    want = [p["C"].clone() for p in probs]
    for p, w in zip(probs, want):
        assert np.array_equal(w.cpu().numpy().view(np.uint16), p["out"].view(np.uint16))
    for policy in ("seq", "ms"):
        for p in probs:
            p["C"].fill_(float("nan"))
        torch.cuda.synchronize()
        run = harness.launch_policy(probs, policy, lib)
        for _ in range(3):
            run()
        torch.cuda.synchronize()
        assert len(harness._runs_of_equal_format(probs)) >= 6              # the problem list alternates formats: several launches
        for p, w in zip(probs, want):
            assert torch.equal(p["C"], w), f"{policy}: {p['size']} {p['q']}"


def test_function_type_call_with_exactly_fifteen_arguments():
    """The registry loop of the reference's test program (mxmoe/kernels/src/test.cu:793-815) on this library: every kernel that
    covers the formats is fetched as a FuncType function and called with that type's 15 arguments, on the stream given to
    mxmoe_set_stream; outputs equal the oracle's bit for bit."""
    import ctypes as C

    from mxmoe_amd import _lib, ops

    lib = _lib.load()
    probs = _mixed_problems(np.random.default_rng(23))
    n = len(probs)
    Cs = [torch.full(p["size"][:2], float("nan"), dtype=torch.float16, device=DEV) for p in probs]
    table = torch.tensor([[p["A"].data_ptr() for p in probs], [p["B"].data_ptr() for p in probs], [p["sa"].data_ptr() for p in probs],
                          [p["sb"].data_ptr() for p in probs], [c.data_ptr() for c in Cs]], dtype=torch.int64).to(DEV)
    row = lambda i: table.data_ptr() + 8 * n * i  # noqa: E731
    h_sizes = (_lib.Dim3 * n)(*[_lib.Dim3(*p["size"]) for p in probs])
    h_q = (_lib.QParams * n)(*[_lib.QParams(p["q"][0], p["q"][1], p["q"][2], 1) for p in probs])
    d_sizes = torch.tensor([list(p["size"]) for p in probs], dtype=torch.int32).to(DEV)
    d_q = torch.frombuffer(bytearray(bytes(h_q)), dtype=torch.uint8).to(DEV)
    side = torch.cuda.Stream()
    ran = 0
    for kid in range(lib.mxmoe_num_kernels()):
        name = lib.mxmoe_kernel_name(kid).decode()
        if "w4a4_g-1_sym" not in name or "w8a8_g-1_sym" not in name or ops.kernel_variants(lib, kid):   # (kernels with operand variants take bf6 fragments / fp8 codes)
            continue
        fn = _lib.FUNC_TYPE(lib.mxmoe_kernel_func(kid))
        for c in Cs:
            c.fill_(float("nan"))
        torch.cuda.synchronize()
        lib.mxmoe_set_stream(side.cuda_stream)
        fn(row(0), row(1), row(2), row(3), row(4), row(4), None, None, None, None, d_sizes.data_ptr(), h_sizes, d_q.data_ptr(), h_q, n)
        lib.mxmoe_set_stream(None)
        assert lib.mxmoe_last_status() == 0, lib.mxmoe_last_error()
        side.synchronize()
        for p, c in zip(probs, Cs):
            assert np.array_equal(c.cpu().numpy().view(np.uint16), p["out"].view(np.uint16)), f"{name}: {p['size']} {p['q']}"
        ran += 1
    assert ran >= 4                                                         # wxax, all, seq_launch_all, ms_launch_all


def test_bench_harness_on_a_workload_file_and_a_legacy_file(tmp_path, capsys):
    """The program the CLI ends in (test.cu:693-946): a synthetic DeepSeek-V2-Lite-shaped trace and qconfig -> workload file ->
    `check`, then `bench` with the default library: one CSV per problem list, named `<output>-<case>-<gate_up|down>.csv`
    (test.cu:942) with the header `kernel_name,avg_time,TFLOPS,speedup` (test.cu:858) and one line per kernel that covers the
    formats; the same through a legacy text input."""
    import json

    from mxmoe_amd import _lib, harness, synth
    from mxmoe_amd.kernels import gen_workload

    cfg = synth.get_config("c4")
    trace, qcfg, wl = tmp_path / "moe-gate.json", tmp_path / "q-wbits4.json", tmp_path / "w.json"
    trace.write_text(json.dumps(synth.trace_dict(cfg)))
    qcfg.write_text(json.dumps(synth.qconfig_dict(cfg)))
    gen_workload.generate_workload_from_gate_trace(str(trace), cfg.tokens, 0, str(wl), str(qcfg), exact_counts=True)
    lib = _lib.load()
    harness.bench_input_file(str(wl), None, lib=lib, mode="check", filters=("groupgemm_hz_fused_wo",))
    assert "max abs err vs fp16 reference" in capsys.readouterr().out
    prefix = str(tmp_path / "bench" / "ds2-synthetic-32")
    (tmp_path / "bench").mkdir()
    res = harness.bench_input_file(str(wl), prefix, lib=lib, mode="bench")
    assert set(res) == {("layer-0", "gate_up"), ("layer-0", "down")}
    for which in ("gate_up", "down"):
        lines = (tmp_path / "bench" / f"ds2-synthetic-32-layer-0-{which}.csv").read_text().splitlines()
        assert lines[0] == "kernel_name,avg_time,TFLOPS,speedup"
        names = [ln.split('",')[0].strip('"') for ln in lines[1:]]
        assert any(n.endswith("groupgemm_hz_fused_wo") for n in names) and any(n.endswith("groupgemm_hz_fused_all") for n in names)
        for ln in lines[1:]:
            ms, tf, sp = (float(x) for x in ln.rsplit('",', 1)[1].split(","))
            assert ms > 0 and tf > 0 and sp > 0
        r = res[("layer-0", which)]
        assert {"fp16-baseline", "mxmoe-hz", "mxmoe-seq", "mxmoe-ms"} <= set(r) and abs(r["mxmoe-hz"][0] - min(float(ln.rsplit('",', 1)[1].split(",")[0]) for ln in lines[1:])) < 1e-4
    legacy = tmp_path / "cases.txt"
    legacy.write_text("4-4--1-sym 300x512x256\n8-8--1-sym 64x256x128\n")
    res = harness.bench_input_file(str(legacy), str(tmp_path / "bench" / "legacy"), lib=lib, mode="bench", filters=("groupgemm_hz_fused_wxax",))
    assert list(res) == [("test_case", "gate_up")]
    assert (tmp_path / "bench" / "legacy-test_case-gate_up.csv").read_text().splitlines()[0] == "kernel_name,avg_time,TFLOPS,speedup"
