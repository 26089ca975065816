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
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(run, [["hipcc", *compile_flags, *extra, *inc, "-Rpass-analysis=kernel-resource-usage", "-c", str(s), "-o", str(o)] for s, o in zip(sources, objs)]))
    run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(out)])
    for o in objs:
        o.unlink()
    objdir.rmdir()
    return out


def build_default(verbose: bool = False) -> Path:
    """Compile every .hip translation unit of the package into libmxmoe_amd.so."""
    sources = sorted(CSRC.glob("*.hip"))
    return hipcc_build(sources, LIB, verbose=verbose)


if __name__ == "__main__":
    print(build_default(verbose=True))
