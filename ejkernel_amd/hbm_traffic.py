"""Turns the FETCH_SIZE / WRITE_SIZE counter files of a rocprofv3 run into HBM bytes per launch.

``python -m ejkernel_amd.hbm_traffic --workload NAME --fetch DIR --write DIR`` reads the ``*counter_collection.csv``
files that ``rocprofv3 --pmc FETCH_SIZE -d DIR ...`` and ``rocprofv3 --pmc WRITE_SIZE -d DIR ...`` left (one counter per
run: the hardware cannot hold both), averages the counters over the dispatches of the attention kernel, scales each
by what the same counter reads for a plain device copy of known size (``bench.py --copy-probe``: FETCH_SIZE counts half
the KiB actually read on MI355X, WRITE_SIZE all of them) and records the result under the workload's name in
``profiles/hbm_traffic.json``, where ``bench.py`` finds ``roofline.traffic``.
"""

from __future__ import annotations

import argparse
import csv
import glob
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def counter_mean(directory: str, counter: str, kernel: str, skip: int = 1) -> float:
    """Mean of `counter` (KiB per dispatch) over the dispatches of kernels whose name contains `kernel`, the first
    `skip` of them (warm-up) left out."""
    vals = []
    for path in sorted(glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)):
        with open(path) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] == counter and kernel in row["Kernel_Name"]:
                    vals.append(float(row["Counter_Value"]))
    if len(vals) <= skip:
        raise SystemExit(f"no {counter} values for a kernel matching {kernel!r} under {directory}")
    vals = vals[skip:]
    return sum(vals) / len(vals)


def record(workload: str, fetch_kib: float, write_kib: float, fetch_scale: float, write_scale: float, command: str) -> dict:
    entry = {"fetch_size_kib": fetch_kib, "write_size_kib": write_kib, "fetch_scale": fetch_scale,
             "write_scale": write_scale, "bytes": (fetch_kib * fetch_scale + write_kib * write_scale) * 1024.0,
             "command": command}
    data = {}
    if os.path.exists(TRAFFIC_FILE):
        with open(TRAFFIC_FILE) as f:
            data = json.load(f)
    data[workload] = entry
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
        f.write("\n")
    return entry


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--workload", required=True)
    ap.add_argument("--fetch", required=True, help="output directory of the FETCH_SIZE run")
    ap.add_argument("--write", required=True, help="output directory of the WRITE_SIZE run")
    ap.add_argument("--kernel", default="rpa_tile_kernel")
    ap.add_argument("--fetch-scale", type=float, default=2.0)
    ap.add_argument("--write-scale", type=float, default=1.0)
    a = ap.parse_args()
    cmd = (f"rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv -d DIR -- python3 bench.py --workload {a.workload} "
           f"--steps 5 --warmup 1 --no-cpu-baseline --no-parity --no-configs")
    e = record(a.workload, counter_mean(a.fetch, "FETCH_SIZE", a.kernel), counter_mean(a.write, "WRITE_SIZE", a.kernel),
               a.fetch_scale, a.write_scale, cmd)
    print(json.dumps({a.workload: e}))


if __name__ == "__main__":
    main()
