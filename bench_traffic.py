#!/usr/bin/env python3
"""Turns rocprofv3 counter runs of bench.py into an entry of profiles/traffic.json.

    rocprofv3 --pmc FETCH_SIZE -d out/fetch -o p --output-format csv -- \\
        python3 bench.py --workload C5 --batch 1 --steps 40 --warmup 5 --no-extra --no-cpu --calibrate-copy
    rocprofv3 --pmc WRITE_SIZE -d out/write -o p --output-format csv -- \\
        python3 bench.py --workload C5 --batch 1 --steps 40 --warmup 5 --no-extra --no-cpu --calibrate-copy
    python3 bench_traffic.py --workload C5 --batch 1 --kernel sp_gemv_i8mfma --fetch out/fetch --write out/write

FETCH_SIZE / WRITE_SIZE are read per dispatch.  The dispatches of the dominant layer are those of the named kernel
whose reading is within 20 % of that kernel's largest (the other layers of the net are smaller).  Each counter is scaled
by what it reads for the plain copy of the net's largest array that --calibrate-copy makes in the same run (a copy
kernel reads and writes exactly that many bytes).  bytes = fetch + write of one launch (times --launches for a batch that
runs in blocks of rows), what bench.py reports as roofline.traffic.  No GPU is needed to run this script.
"""
from __future__ import annotations

import argparse
import csv
import glob
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))


def readings(directory: str, counter: str):
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {directory}")
    rows = []
    for f in files:
        with open(f) as fh:
            for r in csv.DictReader(fh):
                if r["Counter_Name"] == counter:
                    rows.append((r["Kernel_Name"], float(r["Counter_Value"])))
    return rows


def dominant(rows, kernel: str):
    """Mean reading and count of the dominant layer's launches: among the dispatches of `kernel`, the group (same
    instantiation, readings within a few percent) that was launched most often.  bench.py times the dominant layer with
    many extra launches of its own, so it outnumbers every other layer that runs a kernel of the same name."""
    import math
    groups = {}
    for k, v in rows:
        if kernel in k:
            groups.setdefault((k, round(math.log(max(v, 1e-9)) * 16)), []).append(v)
    if not groups:
        raise SystemExit(f"no dispatch of {kernel} in the counter files")
    vals = max(groups.values(), key=lambda g: (len(g), sum(g)))
    return sum(vals) / len(vals), len(vals)


def copy_reading(rows):
    vals = [v for k, v in rows if "copyBuffer" in k or "copy_buffer" in k.lower()]
    if not vals:
        raise SystemExit("no copy kernel dispatch found (run bench.py with --calibrate-copy)")
    return max(vals)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", required=True)
    ap.add_argument("--batch", type=int, required=True)
    ap.add_argument("--kernel", required=True, help="name as sphip_layer_kernel_name reports it")
    ap.add_argument("--fetch", required=True, help="directory of the FETCH_SIZE run")
    ap.add_argument("--write", required=True, help="directory of the WRITE_SIZE run")
    ap.add_argument("--launches", type=int, default=1,
                    help="launches of the kernel per forward of the layer (a batch that runs in blocks of rows: bench.py "
                         "reports it as roofline_kernel.launches); the entry holds their sum")
    ap.add_argument("--no-alt", action="store_true", help="the counter runs were made with bench.py --no-alt (recorded in the entry's commands)")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles", "traffic.json"))
    args = ap.parse_args()

    sys.path.insert(0, ROOT)
    import numpy as np
    from bench import WORKLOADS, BITS  # shapes only; nothing is run
    cfg = WORKLOADS[args.workload]
    topo, prec = cfg["topo"], cfg["prec"]
    l = 1 + int(np.argmax([topo[i] * topo[i + 1] for i in range(len(topo) - 1)]))
    K, N = topo[l - 1], topo[l]
    copy_bytes = max((topo[i] * topo[i + 1] * BITS[prec] + 7) // 8 for i in range(len(topo) - 1))

    fetch_rows, write_rows = readings(args.fetch, "FETCH_SIZE"), readings(args.write, "WRITE_SIZE")
    fetch, nf = dominant(fetch_rows, args.kernel)
    write, _ = dominant(write_rows, args.kernel)
    f_factor = copy_bytes / 1024.0 / copy_reading(fetch_rows)      # KiB of real traffic per counter unit
    w_factor = copy_bytes / 1024.0 / copy_reading(write_rows)
    entry = {
        "kernel": args.kernel, "shape": [args.batch, N, K], "workload": args.workload, "batch": args.batch,
        "fetch_per_dispatch": round(fetch, 1), "write_per_dispatch": round(write, 1), "dispatches_averaged": nf,
        "fetch_factor_kib": round(f_factor, 4), "write_factor_kib": round(w_factor, 4),
        "calibration_copy_bytes": copy_bytes,
        "launches_per_forward": args.launches,
        "bytes": int(round((fetch * f_factor + write * w_factor) * 1024)) * args.launches,
        "commands": [
            f"rocprofv3 --pmc {c} -d out/{d} -o p --output-format csv -- python3 bench.py --workload {args.workload} "
            f"--batch {args.batch} --steps 40 --warmup 5 --no-extra --no-cpu{' --no-alt' if args.no_alt else ''} --calibrate-copy"
            for c, d in (("FETCH_SIZE", "fetch"), ("WRITE_SIZE", "write"))
        ] + [f"python3 bench_traffic.py --workload {args.workload} --batch {args.batch} --kernel {args.kernel} "
             "--fetch out/fetch --write out/write" + (f" --launches {args.launches}" if args.launches > 1 else "") +
             (" --no-alt" if args.no_alt else "")],
    }
    try:
        with open(args.out) as f:
            doc = json.load(f)
    except (OSError, ValueError):
        doc = {"note": "HBM-side bytes per launch of the dominant kernel of each benchmark row; written by bench_traffic.py",
               "entries": []}
    doc["entries"] = [e for e in doc["entries"] if not (e["kernel"] == entry["kernel"] and e["shape"] == entry["shape"])]
    doc["entries"].append(entry)
    doc["entries"].sort(key=lambda e: (e["workload"], e["batch"]))
    with open(args.out, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print(json.dumps(entry))


if __name__ == "__main__":
    main()
