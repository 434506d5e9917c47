"""Turn two rocprofv3 counter runs of bench.py into the HBM traffic record that bench.py reports.

rocprofv3 cannot be driven from inside the benchmarked process, so the bytes a GEMM launch
moves to and from HBM come from two separate runs of the same command, one per counter
(the two do not fit one pass):

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --pmc FETCH_SIZE --kernel-trace -d OUT/fetch -o bench --output-format csv -- \\
        python3 REPO/bench.py --steps 5 --warmup 2 --ramp 3 --no-cpu --no-e4m3 --calib-copy [--config N]
    rocprofv3 --pmc WRITE_SIZE --kernel-trace -d OUT/write -o bench --output-format csv -- \\
        python3 REPO/bench.py --steps 5 --warmup 2 --ramp 3 --no-cpu --no-e4m3 --calib-copy [--config N]
    python3 -m segquant_amd.profile_counters OUT/fetch OUT/write --config N

``--calib-copy`` makes bench.py launch one plain 256 MiB -> 256 MiB elementwise pass (int32 times one); what each
counter reads for that copy gives the counter's unit (the factor to KiB).  The result is merged
into ``profiles/gemm_hbm_traffic_configs_1_to_5.txt`` under the configuration's number; bench.py copies it into its
``roofline`` object as ``traffic`` with ``traffic_source`` saying where it came from.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OUT = os.path.join(ROOT, "profiles", "gemm_hbm_traffic_configs_1_to_5.txt")
COPY_KIB = 256 * 1024  # the yardstick copy reads and writes this many KiB


def _per_kernel(path: str, counter: str):
    files = glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {path}")
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(files[0])):
        if r["Counter_Name"] == counter:
            agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    return agg


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("fetch_dir")
    ap.add_argument("write_dir")
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--kernel", default="gemm", help="substring of the kernel names to sum over (default: the GEMM kernels)")
    args = ap.parse_args()
    rec = {}
    total = 0.0
    launches = None
    for counter, path in (("FETCH_SIZE", args.fetch_dir), ("WRITE_SIZE", args.write_dir)):
        agg = _per_kernel(path, counter)
        # the yardstick is the only int32 multiply-by-a-scalar in the run
        copy = [v for k, vs in agg.items() if "MulFunctor<int>" in k for v in vs]
        if len(copy) != 1:
            raise SystemExit(f"{counter}: expected one yardstick copy in the trace, found {len(copy)} (was bench.py run with --calib-copy?)")
        factor = COPY_KIB / max(copy)  # counter units -> KiB
        kern = {k: vs for k, vs in agg.items() if args.kernel in k}
        n = sum(len(vs) for vs in kern.values())
        kib = sum(sum(vs) for vs in kern.values()) * factor
        rec[counter] = {"factor_to_KiB": round(factor, 3), "KiB_per_launch": round(kib / max(n, 1), 1),
                        "kernels": {k.split("(")[0][-90:]: len(vs) for k, vs in kern.items()}}
        total += kib / max(n, 1) * 1024
        launches = n
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        head = ""
    data = json.load(open(OUT)) if os.path.exists(OUT) else {}
    data[str(args.config)] = {"traffic_bytes_per_launch": round(total), "launches": launches, "counters": rec, "commit": head,
                              "command": "rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --kernel-trace -- python3 bench.py --steps 5 --warmup 2 "
                                         f"--ramp 3 --no-cpu --no-e4m3 --calib-copy --config {args.config}"}
    json.dump(data, open(OUT, "w"), indent=1, sort_keys=True)
    print(json.dumps(data[str(args.config)], indent=1))


if __name__ == "__main__":
    main()
