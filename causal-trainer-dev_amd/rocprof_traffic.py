"""Turns two ``rocprofv3 --pmc`` runs of bench.py into HBM bytes per kernel launch.

Usage (after the two counter runs, each started with ``--calibration-copy-bytes N``)::

    python -m causal_trainer_dev_amd.rocprof_traffic FETCH_DIR WRITE_DIR N [--out profiles]

``FETCH_DIR`` / ``WRITE_DIR`` are the rocprofv3 output folders of the FETCH_SIZE and the
WRITE_SIZE run. Both counters are reported in KiB-like units per dispatch that are not exact
bytes; the plain copy kernel of known size (N bytes read, N bytes written) launched in the same
run gives the factor that converts them. Writes ``traffic.json`` (read by bench.py) and a short
text summary into ``--out``.
"""

from __future__ import annotations

import argparse
import re
import collections
import csv
import glob
import json
import os
import sys

COPY_KERNEL = "ct_calibration_copy_kernel"


def _short(name: str) -> str:
    # counter runs may report the mangled name: _ZN2ct<len><kernel name>I...E...
    mangled = re.match(r"_ZN2ct(\d+)", name)
    if mangled:
        start = mangled.end()
        return name[start:start + int(mangled.group(1))]
    name = name.split("(")[0].replace("void ", "").strip()
    name = name.split("<")[0]
    return name.split("::")[-1]


def read_counter(folder: str, counter: str) -> dict[str, list[float]]:
    """kernel -> list of per-dispatch counter values (summed over the counter's instances)."""

    files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no counter_collection.csv under {folder}")
    per_dispatch = collections.defaultdict(float)
    names = {}
    for path in files:
        with open(path, newline="") as handle:
            for row in csv.DictReader(handle):
                if row["Counter_Name"] != counter:
                    continue
                key = (path, row["Dispatch_Id"])
                per_dispatch[key] += float(row["Counter_Value"])
                names[key] = _short(row["Kernel_Name"])
    result = collections.defaultdict(list)
    for key, value in per_dispatch.items():
        result[names[key]].append(value)
    return result


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    parser.add_argument("fetch_dir")
    parser.add_argument("write_dir")
    parser.add_argument("copy_bytes", type=int)
    parser.add_argument("--out", default="profiles")
    parser.add_argument("--command", default="", help="the rocprofv3 command line, recorded in the summary")
    args = parser.parse_args(argv)

    fetch = read_counter(args.fetch_dir, "FETCH_SIZE")
    write = read_counter(args.write_dir, "WRITE_SIZE")
    if COPY_KERNEL not in fetch or COPY_KERNEL not in write:
        raise SystemExit("the calibration copy kernel is missing from the counter output")
    fetch_factor = args.copy_bytes / (sum(fetch[COPY_KERNEL]) / len(fetch[COPY_KERNEL]))
    write_factor = args.copy_bytes / (sum(write[COPY_KERNEL]) / len(write[COPY_KERNEL]))

    kernels = {}
    for name in sorted(set(fetch) | set(write)):
        if name == COPY_KERNEL or name not in fetch or name not in write:
            continue
        f_mean = sum(fetch[name]) / len(fetch[name])
        w_mean = sum(write[name]) / len(write[name])
        kernels[name] = {
            "fetch_bytes": f_mean * fetch_factor, "write_bytes": w_mean * write_factor,
            "dispatches": len(fetch[name]),
        }
    summary = {
        "copy_bytes": args.copy_bytes,
        "bytes_per_fetch_size_unit": fetch_factor,
        "bytes_per_write_size_unit": write_factor,
        "command": args.command,
        "kernels": kernels,
    }
    os.makedirs(args.out, exist_ok=True)
    with open(os.path.join(args.out, "traffic.json"), "w") as handle:
        json.dump(summary, handle, indent=1, sort_keys=True)
    lines = ["HBM traffic per kernel launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE",
             f"command: {args.command}",
             f"calibration: plain copy of {args.copy_bytes} bytes -> {fetch_factor:.1f} bytes per FETCH_SIZE unit, "
             f"{write_factor:.1f} bytes per WRITE_SIZE unit",
             "", f"{'kernel':36s} {'dispatches':>10s} {'fetch MB':>12s} {'write MB':>12s}"]
    for name, entry in kernels.items():
        lines.append(f"{name:36s} {entry['dispatches']:10d} {entry['fetch_bytes'] / 1e6:12.1f} "
                     f"{entry['write_bytes'] / 1e6:12.1f}")
    text = "\n".join(lines) + "\n"
    with open(os.path.join(args.out, "traffic_bench_attention_cutce.txt"), "w") as handle:
        handle.write(text)
    sys.stdout.write(text)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
