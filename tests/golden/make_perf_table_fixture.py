"""Writes tests/golden/perf_table_sm89_excerpt.json: an excerpt of the reference's kernel-profile table (data file
perf/performance_table.json of the reference checkout), used to test the table consumer against the reference's schema and keys.

Run in a container that has the reference at /root/reference:  python tests/golden/make_perf_table_fixture.py
Only JSON is read; nothing of the reference is imported or executed.
"""
import json
from pathlib import Path

SRC = Path("/root/reference/perf/performance_table.json")
OUT = Path(__file__).resolve().parent / "perf_table_sm89_excerpt.json"
KEEP = {"w8a8_g-1_sym": ["3"], "w4a4_g-1_sym": ["3"], "w4a16_g128_asym": ["1"], "w2a16_g128_asym_accfp16": ["1"]}

table = json.loads(SRC.read_text())
out = {"qcfgs": sorted(table), "slots": {q: sorted(table[q]) for q in table}, "entries": {}}
for q, slots in KEEP.items():
    out["entries"][q] = {s: dict(list(table[q][s].items())[:4]) for s in slots}
OUT.write_text(json.dumps(out, indent=1))
print(OUT, OUT.stat().st_size)
