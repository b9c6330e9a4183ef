"""Turns two rocprofv3 counter runs into the HBM-traffic figure of the attention kernel that bench.py reports.

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/fetch_c2 -o p -- python3 <repo>/bench.py --workload c2 --steps 3 --warmup 1 --no-cpu-baseline --copy-calibration
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir>/write_c2 -o p -- python3 <repo>/bench.py --workload c2 --steps 3 --warmup 1 --no-cpu-baseline --copy-calibration
    python -m baselinebenchmark_amd.benchmarks.traffic_profile --runs <dir> --workloads c2 [c1 c3 c4 ...]

For every workload it averages FETCH_SIZE and WRITE_SIZE (KiB per dispatch, summed over the counter's instances) over
the launches of sage::attn_kernel, scales each by what the same counter reads for the 512 MiB device-to-device copies
that `--copy-calibration` appends to the run (`__amd_rocclr_copyBuffer`, a kernel of known traffic: 524 288 KiB read,
524 288 KiB written; on MI355X FETCH_SIZE reads half of the KiB fetched and WRITE_SIZE all of the KiB written), and
writes profiles/attn_kernel_traffic.json together with the sha256 of the kernel sources the runs were made on
(bench.py prints `traffic: null` when the sources have changed since).
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
COPY_KIB = 512 * 1024.0


def _counter_means(run_dir: str, counter: str):
    """(mean per attention launch, mean per copy launch) of `counter` in a rocprofv3 csv run."""
    files = glob.glob(os.path.join(run_dir, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no *counter_collection.csv under {run_dir}")
    per_dispatch = collections.defaultdict(float)
    kind = {}
    for f in files:
        for r in csv.DictReader(open(f)):
            if r["Counter_Name"] != counter:
                continue
            key = (f, r["Dispatch_Id"])
            per_dispatch[key] += float(r["Counter_Value"])
            name = r["Kernel_Name"]
            # the calibration copy of bench.py (same dtype, contiguous) runs as the runtime's own copy kernel
            kind[key] = "attn" if "attn_kernel" in name else "copy" if "rocclr_copyBuffer" in name else "other"
    attn = [v for k, v in per_dispatch.items() if kind[k] == "attn"]
    copy = [v for k, v in per_dispatch.items() if kind[k] == "copy" and v > 1024.0]   # (not the few-byte copies of scalars)
    if not attn or not copy:
        raise SystemExit(f"{run_dir}: {len(attn)} attention launches and {len(copy)} copy launches found for {counter}")
    return sum(attn) / len(attn), sum(copy) / len(copy), len(attn)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--runs", required=True, help="directory holding fetch_<workload>/ and write_<workload>/ rocprofv3 outputs")
    ap.add_argument("--workloads", nargs="+", default=["c2"])
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles", "attn_kernel_traffic.json"))
    args = ap.parse_args(argv)
    sys.path.insert(0, ROOT)
    import bench
    doc = {"kernel": "sage::attn_kernel", "kernel_source_sha256": bench.kernel_source_digest(),
           "counters": "rocprofv3 --pmc FETCH_SIZE / --pmc WRITE_SIZE, KiB per dispatch, one pass each",
           "calibration": "512 MiB device-to-device copy in the same run: factor = 524288 KiB / counter value of the copy",
           "command": "rocprofv3 --pmc <counter> --output-format csv -d <dir> -o p -- python3 bench.py --workload <w> --steps 3 "
                      "--warmup 1 --no-cpu-baseline --copy-calibration",
           "workloads": {}}
    for w in args.workloads:
        fetch, fetch_copy, n = _counter_means(os.path.join(args.runs, f"fetch_{w}"), "FETCH_SIZE")
        write, write_copy, _ = _counter_means(os.path.join(args.runs, f"write_{w}"), "WRITE_SIZE")
        ff, wf = COPY_KIB / fetch_copy, COPY_KIB / write_copy
        doc["workloads"][w] = {"launches": n, "fetch_kib": fetch, "write_kib": write, "fetch_factor": ff, "write_factor": wf,
                               "bytes": (fetch * ff + write * wf) * 1024.0}
        print(f"{w}: FETCH_SIZE {fetch:.0f} x {ff:.3f}, WRITE_SIZE {write:.0f} x {wf:.3f} -> {doc['workloads'][w]['bytes'] / 1e9:.3f} GB per launch")
    with open(args.out, "w") as f:
        json.dump(doc, f, indent=1)
        f.write("\n")
    print(f"wrote {args.out}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
