"""HBM traffic of the headline matvec kernel from hardware counters, as a small record that bench.py reads.

    python -m skainet_amd.traffic --fetch mv_fetch.csv --write mv_write.csv --copy-fetch cp_fetch.csv \\
        --copy-write cp_write.csv -o profiles/matvec_q4k_4096x11008_traffic.json

The four inputs are the `*_counter_collection.csv` files of four rocprofv3 runs (one counter per run):

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o p -- python3 bench.py --steps 200 --warmup 10 --no-cpu --no-extra
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out -o p -- python3 bench.py --steps 200 --warmup 10 --no-cpu --no-extra
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d out -o p -- python3 bench.py --mode copy --steps 200
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d out -o p -- python3 bench.py --mode copy --steps 200

The copy kernel moves a known number of bytes, which calibrates the counters' units; the record also carries a hash of
the kernel's sources, and bench.py reports the traffic only while that hash still matches the tree it runs from.
"""
from __future__ import annotations

import argparse
import csv
import hashlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_SOURCES = ("csrc/matvec.hip", "csrc/common.h", "csrc/kv.h")
HEADLINE_KERNEL = "matvec_q4k_kernel"
COPY_KERNEL = "copy16_kernel"
COPY_BYTES = 4096 * (11008 // 256) * 144  # what `bench.py --mode copy` reads and writes per launch


def source_hash() -> str:
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(HERE, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def counter_mean(path: str, kernel: str, counter: str):
    """Mean, minimum, maximum and count of `counter` over the dispatches of `kernel` in a rocprofv3 counter CSV."""
    vals = []
    with open(path, newline="") as f:
        for row in csv.DictReader(f):
            if row["Counter_Name"] == counter and kernel in row["Kernel_Name"]:
                vals.append(float(row["Counter_Value"]))
    if not vals:
        raise ValueError(f"{path}: no {counter} rows for a kernel named *{kernel}*")
    return sum(vals) / len(vals), min(vals), max(vals), len(vals)


def build_record(fetch_csv, write_csv, copy_fetch_csv, copy_write_csv):
    mf = counter_mean(fetch_csv, HEADLINE_KERNEL, "FETCH_SIZE")
    mw = counter_mean(write_csv, HEADLINE_KERNEL, "WRITE_SIZE")
    cf = counter_mean(copy_fetch_csv, COPY_KERNEL, "FETCH_SIZE")
    cw = counter_mean(copy_write_csv, COPY_KERNEL, "WRITE_SIZE")
    fetch_unit, write_unit = COPY_BYTES / cf[0], COPY_BYTES / cw[0]  # bytes per count
    read_b, written_b = mf[0] * fetch_unit, mw[0] * write_unit
    return {
        "kernel": HEADLINE_KERNEL,
        "workload": "Q4_K matvec N=4096 K=11008, weights rotating over 24 copies",
        "source_hash": source_hash(),
        "counters_per_dispatch": {
            "matvec_FETCH_SIZE": {"mean": mf[0], "min": mf[1], "max": mf[2], "dispatches": mf[3]},
            "matvec_WRITE_SIZE": {"mean": mw[0], "min": mw[1], "max": mw[2], "dispatches": mw[3]},
            "copy_FETCH_SIZE": {"mean": cf[0], "min": cf[1], "max": cf[2], "dispatches": cf[3]},
            "copy_WRITE_SIZE": {"mean": cw[0], "min": cw[1], "max": cw[2], "dispatches": cw[3]},
        },
        "copy_bytes_each_way": COPY_BYTES,
        "bytes_per_count": {"FETCH_SIZE": fetch_unit, "WRITE_SIZE": write_unit},
        "read_bytes": round(read_b),
        "written_bytes": round(written_b),
        "traffic_bytes": round(read_b + written_b),
    }


def load_current(path):
    """The record at `path` if it was taken on the kernel sources of this tree, else None."""
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    return rec if rec.get("source_hash") == source_hash() else None


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--copy-fetch", required=True)
    ap.add_argument("--copy-write", required=True)
    ap.add_argument("-o", "--out", required=True)
    a = ap.parse_args()
    rec = build_record(a.fetch, a.write, a.copy_fetch, a.copy_write)
    with open(a.out, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
