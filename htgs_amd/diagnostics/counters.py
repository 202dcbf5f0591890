"""Turns rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs into the HBM-traffic record that ``bench.py`` reports.

    python -m htgs_amd.diagnostics.counters --key cfg2/mode0/K16/rasterize --kernel blend_hybrid_kernel \\
        --fetch F_results.db --write W_results.db --cal-fetch CF_results.db --cal-write CW_results.db [--table]

Each ``*_results.db`` is the sqlite file of one ``rocprofv3 --pmc <counter> -d DIR -o NAME -- python3 bench.py ...`` run
(one counter per run).  The two calibration runs are the same counters over ``bench.py --calibrate`` (a plain copy of
1 GiB each way): the counters' units differ from generation to generation, so every reading is scaled by what the same
counter shows for a known number of bytes.  The result goes to ``profiles/counters.json`` together with the digest of the
kernel sources it was measured on; ``bench.py`` reports the figure only while that digest matches the tree.
"""
from __future__ import annotations

import argparse
import collections
import json
import os
import sqlite3
import statistics

from ..build import csrc_digest

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
COUNTERS_FILE = os.path.join(ROOT, "profiles", "counters.json")
CAL_KERNEL, CAL_BYTES = "copy_bytes_kernel", 1 << 30


def short_name(kernel: str) -> str:
    """the kernel's name without its argument list (a name may itself begin with a parenthesis: "(anonymous namespace)::")"""
    return kernel.replace("(anonymous namespace)::", "").split("(")[0].replace("void ", "")


def per_kernel_median(db_path: str, counter: str) -> dict:
    """kernel name (without its argument list) -> median over dispatches of the counter summed over its dimensions"""
    db = sqlite3.connect(db_path)
    rows = db.execute("select kernel_name, dispatch_id, value from counters_collection where counter_name = ?", (counter,)).fetchall()
    per_dispatch = collections.defaultdict(float)
    for name, dispatch, value in rows:
        per_dispatch[(short_name(name), dispatch)] += value
    per_kernel = collections.defaultdict(list)
    for (name, _), value in per_dispatch.items():
        per_kernel[name].append(value)
    return {k: statistics.median(v) for k, v in per_kernel.items()}


def scale_factor(db_path: str, counter: str) -> float:
    med = per_kernel_median(db_path, counter)
    hits = [v for k, v in med.items() if CAL_KERNEL in k]
    if len(hits) != 1 or hits[0] <= 0:
        raise SystemExit(f"{db_path}: no {CAL_KERNEL} dispatch with a {counter} reading")
    return (CAL_BYTES / 1024.0) / hits[0]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--key", required=True, help="workload key, as bench.py builds it: cfg<c>[-n<N>]/mode<m>/K<k>/<rasterize|fast_rasterize|train<rows>>")
    ap.add_argument("--kernel", required=True, help="substring naming the dominant kernel (or kernels: their bytes add up) of that workload")
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--cal-fetch", required=True)
    ap.add_argument("--cal-write", required=True)
    ap.add_argument("--table", action="store_true", help="also print a markdown table of every kernel of the run")
    args = ap.parse_args()

    fs, ws = scale_factor(args.cal_fetch, "FETCH_SIZE"), scale_factor(args.cal_write, "WRITE_SIZE")
    fetch, write = per_kernel_median(args.fetch, "FETCH_SIZE"), per_kernel_median(args.write, "WRITE_SIZE")
    # (the dominant stage of a workload may be two launches -- the kernel with one wave per tile and the one for the tiles
    # with very long lists: every kernel whose name contains the pattern counts, their bytes add up)
    names = sorted(k for k in fetch if args.kernel in k)
    if not names:
        raise SystemExit(f"--kernel {args.kernel!r} matches no kernel of {args.fetch}")
    fetch_kib = sum(fetch[k] for k in names)
    write_kib = sum(write.get(k, 0.0) for k in names)
    read_b, write_b = fetch_kib * 1024.0 * fs, write_kib * 1024.0 * ws
    entry = {"kernel": " + ".join(names), "fetch_KiB": fetch_kib, "write_KiB": write_kib, "fetch_scale": round(fs, 4),
             "write_scale": round(ws, 4), "read_bytes": int(read_b), "written_bytes": int(write_b), "traffic_bytes": int(read_b + write_b)}
    digest = csrc_digest()
    try:
        with open(COUNTERS_FILE) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        rec = {}
    if rec.get("csrc_sha256") != digest:
        rec = {"csrc_sha256": digest, "launches": {}}        # readings of other sources describe other code
    rec["launches"][args.key] = entry
    with open(COUNTERS_FILE, "w") as f:
        json.dump(rec, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({args.key: entry}))
    if args.table:
        print(f"\nscale factors: fetch x {fs:.3f}, write x {ws:.3f}\n")
        print("| kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | scaled read MB | scaled write MB |\n|---|---|---|---|---|")
        for k in fetch:
            if "rocclr" in k or "at::" in k or "elementwise" in k:
                continue
            print(f"| `{k}` | {fetch[k]:.0f} | {write.get(k, 0):.0f} | {fetch[k] * 1024 * fs / 1e6:.1f} | {write.get(k, 0) * 1024 * ws / 1e6:.1f} |")


if __name__ == "__main__":
    main()
