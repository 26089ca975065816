"""Build the gfx950 C-ABI library in-tree with hipcc (no cmake, no JIT cache).

Replaces the reference's CMake + FetchContent build (mxmoe/kernels/src/CMakeLists.txt:44-58,87-116,
mxmoe/kernels/src/setup.py:6-31).  `--use_fast_math` of the reference is deliberately NOT mirrored and FMA
contraction is off: the quantiser and the Hadamard rotation must round exactly like their CPU restatement.
"""
from __future__ import annotations

import re
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "libmxmoe_amd.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-Wno-inline-asm",  # the LDS-DMA helper sets M0 itself
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def check_no_spills(remarks: str) -> None:
    """Refuse a build in which a WxAxTile kernel spills vector registers.

    Those tiles load weight fragments with loads the compiler does not track (the waits are placed by hand): a fragment register
    that the compiler spills or re-uses while its load is in flight is overwritten when the load lands, and when that register
    holds an address the next access faults.  `remarks` is hipcc's -Rpass-analysis=kernel-resource-usage output."""
    name = None
    for line in remarks.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            continue
        m = re.search(r"remark:\s+VGPRs Spill: (\d+)", line)
        if m and name and ("WxAxTile" in name or "Bf6Tile" in name) and int(m.group(1)) > 0:
            raise RuntimeError(f"{name}: {m.group(1)} vector registers spilled in a kernel with hand-tracked loads; shrink the tile's "
                               f"register ring or lower its waves per SIMD")


_VMEM = re.compile(r"(global_|buffer_|flat_|scratch_)(load|store|atomic)")


def check_untracked_load_copies(asm: str) -> None:
    """Refuse device code in which the compiler touches a register while a hand-tracked load into it is in flight, or adds a
    vector-memory instruction of its own where vector-memory instructions are counted by hand.

    The weight fragments of the WxAxTile kernels are loaded by inline-assembly `global_load_dwordx4` whose completion only the
    hand-placed `s_waitcnt vmcnt(N) ; landed v[a:b]` knows about, and N is the exact number of younger vector-memory instructions
    (fragment loads and direct-to-LDS loads, all inline assembly).  `asm` is hipcc's -S output for the device.  Every kernel is
    cut into basic blocks and the set of registers possibly in flight (added by an inline-assembly load, removed by the wait that
    names them) is propagated along its branches to a fixed point, so loads issued at the bottom of a loop iteration are in flight
    at its top and code the compiler lays out elsewhere is judged by how control reaches it.  Refused:

    * ANY compiler-generated instruction (whatever its mnemonic: a move, a spill, a permute, an ordinary ALU operation reading or
      overwriting it) that names a register in flight: it would read stale data, or its result would be overwritten when the load
      lands;
    * any compiler-generated vector-memory instruction, inside a loop or not, while a hand-tracked load is in flight: it would be
      one more instruction in the queue than the hand-computed N assumes;
    * a compiler-generated store, atomic or scratch access while direct-to-LDS loads (inline assembly too, awaited by hand-placed
      counts) may be outstanding, i.e. since the last hand-placed wait for vmcnt(0): writes retire out of order with the loads, so
      a count that includes one says nothing about the loads.  Compiler-generated LOADS are allowed there: loads retire in
      order, so one more younger load makes a hand-placed wait last longer, never shorter (the weight-only MFMA tile counts on
      exactly that: its weight loads are the compiler's, its activation loads go straight to LDS);
    * a load that is never waited for."""
    lines = asm.splitlines()
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\w+:", l)]

    def regs_of(text):
        out = set()
        for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", text):
            out.update(range(int(a), int(b) + 1))
        out.update(int(a) for a in re.findall(r"\bv(\d+)\b", text))
        return out

    for si, start in enumerate(starts):
        end = starts[si + 1] if si + 1 < len(starts) else len(lines)
        end = next((i for i in range(start, end) if lines[i].startswith(".Lfunc_end")), end)
        kernel = lines[start].split(":")[0]
        # basic blocks: (instructions as (line number, text, inside inline assembly), successor labels, falls through)
        blocks, label_of, cur, inside = [], {}, None, False

        def new_block():
            blocks.append({"ins": [], "succ": [], "fall": True})
            return blocks[-1]

        cur = new_block()
        for i in range(start + 1, end):
            raw = lines[i]
            t = raw.strip()
            m = re.match(r"^(\.LBB\d+_\d+):", raw)
            if m:
                if cur["ins"] or cur["succ"] or len(blocks) == 1:
                    cur = new_block()
                label_of[m.group(1)] = len(blocks) - 1
                continue
            if t.startswith(";;#ASMSTART"):
                inside = True
                continue
            if t.startswith(";;#ASMEND"):
                inside = False
                continue
            if not t or t.startswith(";") or t.startswith("."):
                continue
            cur["ins"].append((i, t, inside))
            if inside:
                continue
            m = re.match(r"s_(c?branch)\w*\s+(\.LBB\d+_\d+)", t)
            if m:
                cur["succ"].append(m.group(2))
                cur["fall"] = m.group(1) == "cbranch"
                cur = new_block()
            elif re.match(r"s_(endpgm|setpc_b64|trap)", t):
                cur["fall"] = False
                cur = new_block()

        def successors(b):
            out = [label_of[l] for l in blocks[b]["succ"] if l in label_of]
            if blocks[b]["fall"] and b + 1 < len(blocks):
                out.append(b + 1)
            return out

        # Forward may-analysis over the control-flow graph to a fixed point.  State at a block's entry: registers with a hand-tracked
        # load possibly in flight, and `lds_pending` (direct-to-LDS loads, counted by hand as well but landing in no register, may
        # be outstanding: only a hand-placed wait for vmcnt(0) is known to have drained them).
        state_in = {0: (frozenset(), False)}
        work = [0]
        while work:
            b = work.pop()
            inflight, lds_pending = set(state_in[b][0]), state_in[b][1]
            for i, t, in_asm in blocks[b]["ins"]:
                if in_asm:
                    if t.startswith("global_load"):
                        inflight |= regs_of(t.split(",")[0])
                    elif _VMEM.match(t):
                        lds_pending = True
                    elif t.startswith("s_waitcnt"):
                        if "; landed" in t:
                            inflight -= regs_of(t.split("; landed")[1])
                        if re.search(r"vmcnt\(0\)", t):  # every vector-memory instruction issued so far has completed
                            inflight.clear()
                            lds_pending = False
                elif _VMEM.match(t) and (inflight or (lds_pending and not re.match(r"(global|buffer|flat)_load", t))):
                    raise RuntimeError(f"{kernel}: line {i + 1} `{t}`: compiler-generated vector-memory instruction while vector-memory "
                                       f"instructions are counted by hand (loads in flight: v{sorted(inflight)}, direct-to-LDS loads pending: {lds_pending})")
                elif inflight and regs_of(t.split(";")[0]) & inflight:
                    raise RuntimeError(f"{kernel}: line {i + 1} `{t}` touches a register while a hand-tracked load into it is in flight; "
                                       f"restructure the tile so that no fragment register is live across a branch")
                elif inflight and t.startswith("s_endpgm"):
                    raise RuntimeError(f"{kernel}: hand-tracked loads into v{sorted(inflight)} are never waited for")
            succ = successors(b)
            if inflight and not succ and not any(t.startswith("s_endpgm") for _, t, _ in blocks[b]["ins"]):
                raise RuntimeError(f"{kernel}: hand-tracked loads into v{sorted(inflight)} are never waited for")
            for n in succ:
                old = state_in.get(n)
                new = (frozenset(inflight) | (old[0] if old else frozenset()), lds_pending or (old[1] if old else False))
                if new != old:
                    state_in[n] = new
                    work.append(n)


def hipcc_build(sources, out: Path, extra=(), verbose: bool = False, jobs: int = 8) -> Path:
    """Compile each source to an object (in parallel) and link them into the shared library `out`."""
    from concurrent.futures import ThreadPoolExecutor

    sources = [Path(s) for s in sources]
    out = Path(out)
    objdir = out.parent / f".obj_{out.stem}"
    objdir.mkdir(parents=True, exist_ok=True)
    inc = [f"-I{CSRC / 'include'}", f"-I{PKG.parent / 'include'}"]
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]

    def run(cmd):
        res = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(map(str, cmd))}\n{err}")
        check_no_spills(err)
        err = "\n".join(l for l in err.splitlines() if "kernel-resource-usage" not in l and not re.match(r"\s*(\d+\s*)?\||In file included", l))
        if verbose and err.strip():
            print(err, file=sys.stderr)

    objs = [objdir / (s.stem + ".o") for s in sources]

    def scan(src):
        # device assembly of the same translation unit, only to be checked
        out_s = objdir / (src.stem + ".s")
        run(["hipcc", *[f for f in compile_flags if f != "-fPIC"], *extra, *inc, "-S", "--cuda-device-only", str(src), "-o", str(out_s)])
        try:
            check_untracked_load_copies(out_s.read_text())
        finally:
            out_s.unlink()

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        jobs_ = [ex.submit(run, ["hipcc", *compile_flags, *extra, *inc, "-Rpass-analysis=kernel-resource-usage", "-c", str(s), "-o", str(o)]) for s, o in zip(sources, objs)]
        jobs_ += [ex.submit(scan, s) for s in sources]
        for j in jobs_:
            j.result()
    run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(out)])
    for o in objs:
        o.unlink()
    objdir.rmdir()
    return out


def build_default(verbose: bool = False) -> Path:
    """Compile every .hip translation unit of the package, and the generator's registration unit of the default kernels, into
    libmxmoe_amd.so."""
    from .kernels.compose_kernel import emit_default_library

    sources = sorted(CSRC.glob("*.hip")) + emit_default_library()
    return hipcc_build(sources, LIB, verbose=verbose)


def sample_generator():
    """The generator run whose library ships prebuilt next to the default one: {w4a4, w8a8} with two shapes per format as
    one-tile-per-format combinations (4 kernels) plus one kernel carrying both formats' shape sets.  The GPU tests load it, so
    the flow generator -> hipcc -> registry -> launch is exercised without compiling on the GPU machine."""
    from .kernels.compose_kernel import GEN_DIR, KernelType, TemplateGenerator
    from .kernels.tile_config import get_possible_tile_list

    tiles = {q: [t for t in get_possible_tile_list("gfx950", q) if t.BM in (128, 32) and not t.is_bf6()] for q in ("w4a4_g-1_sym", "w8a8_g-1_sym")}
    for q in tiles:
        tiles[q] = tiles[q] + [tuple(tiles[q])]
    gen = TemplateGenerator("gfx950", list(tiles), KernelType.Fused, tiles, out_dir=GEN_DIR / "sample_w4a4_w8a8")
    combos = [c for c in gen.get_tile_configs() if sum(isinstance(t, tuple) for t in c.values()) in (0, len(c))]
    gen.get_tile_configs = lambda: combos
    return gen


def build_generated_sample(verbose: bool = False) -> Path:
    gen = sample_generator()
    gen.generate_source_code()
    return gen.build()


if __name__ == "__main__":
    print(build_default(verbose=True))
    print(build_generated_sample(verbose=True))
