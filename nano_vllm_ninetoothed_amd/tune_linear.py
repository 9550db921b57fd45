"""Finds, for each (rows, n, k) of a model's decode-step projections, the hipBLASLt solution that is fastest
when the weights are cold, and writes the table `mops.hip.ops.load_linear_solutions` reads.

Usage (on the GPU the table is for):
    python -m nano_vllm_ninetoothed_amd.tune_linear --out nano_vllm_ninetoothed_amd/data/linear_solutions_gfx950.json

The projections are those of nanovllm/models/qwen3.py:39-56,101-117 at the Qwen3-0.6B sizes unless --shapes
gives others as n:k pairs; the row counts default to the engine counterpart's graph batch sizes.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time


def _dump(table: dict) -> str:
    """JSON with one table entry per line."""
    head = {k: v for k, v in table.items() if k not in ("solutions", "timings_us")}
    lines = ["{"] + [f'"{k}": {json.dumps(v)},' for k, v in head.items()]
    for key in ("solutions", "timings_us"):
        lines.append(f'"{key}": [')
        lines += [json.dumps(e) + ("," if i + 1 < len(table[key]) else "") for i, e in enumerate(table[key])]
        lines.append("]," if key == "solutions" else "]")
    lines.append("}")
    return "\n".join(lines) + "\n"


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", required=True)
    ap.add_argument("--shapes", default="4096:1024,1024:2048,6144:1024,1024:3072", help="n:k pairs of the weight matrices")
    ap.add_argument("--rows", default="1,2,4,8," + ",".join(str(b) for b in range(16, 257, 16)))
    ap.add_argument("--layers", type=int, default=28, help="distinct weight matrices cycled through per measurement")
    ap.add_argument("--rounds", type=int, default=2)
    ap.add_argument("--merge", action="store_true", help="keep the entries of an existing --out file for other shapes")
    args = ap.parse_args()

    import torch
    from . import _capi
    lib = _capi.load()
    dev = torch.device("cuda:0")
    ws = torch.empty(32 << 20, dtype=torch.uint8, device=dev)
    shapes = [tuple(int(v) for v in s.split(":")) for s in args.shapes.split(",")]
    rows = [int(r) for r in args.rows.split(",")]
    out = {"hip_version": torch.version.hip, "arch": torch.cuda.get_device_properties(dev).gcnArchName.split(":")[0],
           "note": "hipBLASLt solution index per [rows, n, k], fastest on cold weights; timings_us rows are [rows, n, k, best, heuristic's choice]",
           "solutions": [], "timings_us": []}
    if args.merge and os.path.exists(args.out):
        with open(args.out) as f:
            old = json.load(f)
        if old.get("hip_version") == out["hip_version"] and old.get("arch") == out["arch"]:
            todo = {(m, n, k) for m in rows for n, k in shapes}
            out["solutions"] = [e for e in old["solutions"] if tuple(e[:3]) not in todo]
            out["timings_us"] = [e for e in old["timings_us"] if tuple(e[:3]) not in todo]
    for m in rows:
        for n, k in shapes:
            best, best_us, heur_us = ctypes.c_int(-1), ctypes.c_float(-1), ctypes.c_float(-1)
            t0 = time.time()
            st = lib.mops_hip_linear_tune(m, n, k, args.layers, args.rounds, ws.data_ptr(), ws.numel(),
                                          ctypes.byref(best), ctypes.byref(best_us), ctypes.byref(heur_us))
            _capi.check("mops_hip_linear_tune", st)
            out["solutions"].append([m, n, k, best.value])
            out["timings_us"].append([m, n, k, round(best_us.value, 2), round(heur_us.value, 2)])
            print(f"m={m} n={n} k={k}: solution {best.value} {best_us.value:.2f} us (heuristic's choice {heur_us.value:.2f} us), "
                  f"searched in {time.time() - t0:.1f} s", flush=True)
            with open(args.out, "w") as f:      # rewritten after every shape so that a cut-off run still leaves a table
                f.write(_dump(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
