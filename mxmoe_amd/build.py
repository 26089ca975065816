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
        if m and name and "WxAxTile" in name and int(m.group(1)) > 0:
            raise RuntimeError(f"{name}: {m.group(1)} vector registers spilled in a kernel with hand-tracked loads; shrink the tile's "
                               f"register ring or lower its waves per SIMD")


def check_untracked_load_copies(asm: str) -> None:
    """Refuse device code in which a register is moved by the compiler while a hand-tracked load into it is in flight.

    The weight fragments of the WxAxTile kernels are loaded by inline-assembly `global_load_dwordx4` whose completion only the
    hand-placed `s_waitcnt vmcnt(N) ; landed v[a:b]` knows about.  A register-to-register copy (or a spill) of such a register,
    which the register allocator is free to insert wherever the value is live across a branch or a loop edge, copies whatever the
    register holds at that moment.  `asm` is hipcc's -S output for the device.  Every kernel is walked in layout order with the set
    of registers in flight (added by an inline-assembly load, removed by the wait that names them); loop bodies are walked twice,
    so that loads issued at the bottom of an iteration are in flight at its top."""
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
        kernel = lines[start].split(":")[0]
        # loop regions: header line .. end of the last block that names the header
        label_lines = [i for i in range(start, end) if re.match(r"^\.LBB\d+_\d+:", lines[i])]
        regions = []
        for h in (i for i in range(start, end) if "Loop Header" in lines[i]):
            name = lines[h].split(":")[0].strip().lstrip(".L")
            members = [i for i in range(start, end) if re.search(rf"Header={name}\b", lines[i])]
            last = max([h] + members)
            nxt = next((i for i in label_lines if i > last), end)
            regions.append((min([h] + members), nxt))
        order, pos = [], start
        for lo, hi in sorted(regions):
            if lo < pos:
                continue
            order += list(range(pos, lo)) + list(range(lo, hi)) * 2
            pos = hi
        order += list(range(pos, end))
        # a loop that issues hand-tracked loads counts every vector-memory instruction: the compiler must not add its own there
        for lo, hi in regions:
            body = [lines[i].strip() for i in range(lo, hi)]
            tracked, inside = False, False
            for t in body:
                inside = True if t.startswith(";;#ASMSTART") else False if t.startswith(";;#ASMEND") else inside
                tracked |= inside and t.startswith("global_load")
            inside = False
            for k, t in enumerate(body):
                inside = True if t.startswith(";;#ASMSTART") else False if t.startswith(";;#ASMEND") else inside
                if tracked and not inside and re.match(r"(global_|buffer_|flat_|scratch_)(load|store|atomic)", t):
                    raise RuntimeError(f"{kernel}: line {lo + k + 1} `{t}`: compiler-generated vector-memory instruction inside a loop whose "
                                       f"loads are counted by hand")
        inflight, in_asm = set(), False
        for i in order:
            t = lines[i].strip()
            if t.startswith(";;#ASMSTART"):
                in_asm = True
            elif t.startswith(";;#ASMEND"):
                in_asm = False
            elif in_asm and t.startswith("global_load"):
                inflight |= regs_of(t.split(",")[0])
            elif in_asm and t.startswith("s_waitcnt") and "; landed" in t:
                inflight -= regs_of(t.split("; landed")[1])
            elif not in_asm and inflight and re.match(r"(v_mov_b|v_accvgpr_|scratch_|v_swap_)", t) and regs_of(t) & inflight:
                raise RuntimeError(f"{kernel}: line {i + 1} `{t}` moves a register while a hand-tracked load into it is in flight; "
                                   f"restructure the tile so that no fragment register is live across a branch")
        if inflight:
            raise RuntimeError(f"{kernel}: hand-tracked loads into v{sorted(inflight)} are never waited for")


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

    sources = sorted(CSRC.glob("*.hip")) + [emit_default_library()]
    return hipcc_build(sources, LIB, verbose=verbose)


def sample_generator():
    """The generator run whose library ships prebuilt next to the default one: {w4a4, w8a8} with two shapes per format as
    one-tile-per-format combinations (4 kernels) plus one kernel carrying both formats' shape sets.  The GPU tests load it, so
    the flow generator -> hipcc -> registry -> launch is exercised without compiling on the GPU machine."""
    from .kernels.compose_kernel import GEN_DIR, KernelType, TemplateGenerator
    from .kernels.tile_config import get_possible_tile_list

    tiles = {q: [t for t in get_possible_tile_list("gfx950", q) if t.BM in (128, 32)] for q in ("w4a4_g-1_sym", "w8a8_g-1_sym")}
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
