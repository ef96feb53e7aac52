"""Writes tests/golden/algo_table.json: the 102 twelve-number rows of the Algo
index space, read as text from the reference's generated function-pointer table
(src/tiling/gemm_tiling.cuh:4-105; signal_tiling.cuh and scatter_tiling.cuh list
the same rows).  Run once in the build container, where the reference tree is
mounted; only the JSON travels.

    python tests/golden/make_algo_table.py [/root/reference]
"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
rows = {}
for name in ("gemm_tiling.cuh", "signal_tiling.cuh", "scatter_tiling.cuh"):
    text = open(os.path.join(ref, "src", "tiling", name)).read()
    rows[name] = [[int(v) for v in m.split(",")] for m in re.findall(r"<([0-9, ]+)>", text)]
assert rows["gemm_tiling.cuh"] == rows["signal_tiling.cuh"] == rows["scatter_tiling.cuh"]
table = rows["gemm_tiling.cuh"]
assert all(len(r) == 12 for r in table)
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "algo_table.json")
with open(out, "w") as f:
    json.dump({"fields": ["TbM", "TbN", "TbK", "WarpM", "WarpN", "WarpK", "InstM", "InstN", "InstK",
                          "Stages", "Swizzle", "SplitK"], "rows": table}, f)
print(len(table), "rows ->", out)
