"""Build ``had_tables.npz``: the K x K (+1/-1) Hadamard matrices used for n = K * 2^m sizes.

The matrices are published data (N. J. A. Sloane's Hadamard library, neilsloane.com/hadamard);
the reference keeps them as literal ``+1, -1`` tables in ``mxmoe/quant/hadamard_utils.py:162-4379``
(``get_had12`` ... ``get_had176``).  This script reads that file as *text*, extracts the sign
tables, checks ``H @ H.T == K * I`` for each, and stores them bit-packed (1 bit per entry, bit set
means -1) so the product and the CPU oracle can load them without the reference being present.

Run once, where a checkout of the reference exists; the table file is the argument:
    python mxmoe_amd/data/make_had_tables.py <reference>/mxmoe/quant/hadamard_utils.py
Nothing in the package imports this script or knows where a reference checkout lives.
"""
import re
import sys
from pathlib import Path

import numpy as np

OUT = Path(__file__).with_name("had_tables.npz")


def main() -> int:
    if len(sys.argv) != 2:
        print(__doc__)
        return 2
    text = Path(sys.argv[1]).read_text()
    blocks = re.split(r"^def get_had(\d+)\(\):", text, flags=re.M)
    tables = {}
    for name, body in zip(blocks[1::2], blocks[2::2]):
        k = int(name)
        body = body.split("\ndef ")[0]
        signs = re.findall(r"([+-])\s*1\b", body)
        if len(signs) != k * k:
            print(f"skip had{k}: {len(signs)} entries, expected {k * k}")
            continue
        h = np.array([1 if s == "+" else -1 for s in signs], dtype=np.int32).reshape(k, k)
        gram = h @ h.T
        assert np.array_equal(gram, k * np.eye(k, dtype=np.int32)), f"had{k} is not Hadamard"
        tables[f"had{k}"] = np.packbits((h < 0).astype(np.uint8).reshape(-1))
        print(f"had{k}: ok ({k}x{k})")
    np.savez_compressed(OUT, **tables)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")
    return 0


if __name__ == "__main__":
    sys.exit(main())
