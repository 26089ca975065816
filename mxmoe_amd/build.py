"""Build the gfx950 C-ABI library in-tree with hipcc (no cmake, no JIT cache).

Replaces the reference's CMake + FetchContent build (mxmoe/kernels/src/CMakeLists.txt:44-58,87-116,
mxmoe/kernels/src/setup.py:6-31).  `--use_fast_math` of the reference is deliberately NOT mirrored and FMA
contraction is off: the quantiser and the Hadamard rotation must round exactly like their CPU restatement.
"""
from __future__ import annotations

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
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_build(sources, out: Path, extra=(), verbose: bool = False) -> Path:
    cmd = ["hipcc", *HIPCC_FLAGS, *extra, f"-I{CSRC / 'include'}", f"-I{PKG.parent / 'include'}", *map(str, sources), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(cmd)}\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return out


def build_default(verbose: bool = False) -> Path:
    """Compile every .hip translation unit of the package into libmxmoe_amd.so."""
    sources = sorted(CSRC.glob("*.hip"))
    return hipcc_build(sources, LIB, verbose=verbose)


if __name__ == "__main__":
    print(build_default(verbose=True))
