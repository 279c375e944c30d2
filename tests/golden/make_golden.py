"""Regenerates seed0_totals.json from the workload generator.

The expected values in the committed JSON were first taken from the published
table of known answers for the five configurations (seed 0); this script only
exists to show how the table is reproduced.  Run: python tests/golden/make_golden.py
"""
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from blockedattention_amd import workloads  # noqa: E402

out = {}
for cfg in range(1, 6):
    w = workloads.make(cfg, seed=0)
    out[f"cfg{cfg}"] = {"segments": w.nseg, "heads": w.heads, "rows": int(w.M.sum()), "Dm1": w.Dm1, "Dm2": w.Dm2,
                        "Dout": w.Dout}
out["cfg5"]["n"] = [int(v) for v in workloads.make(5).M]
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "seed0_totals.json")
with open(path, "w") as f:
    json.dump(out, f, indent=1)
print(path)
