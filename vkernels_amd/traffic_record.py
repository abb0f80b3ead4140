"""Turns two rocprofv3 counter runs of bench.py (FETCH_SIZE, then WRITE_SIZE, each with
--copy-calibration) into the record bench.py reports as roofline.traffic.

    python -m vkernels_amd.traffic_record --workload c1:64 --kernel "stream_resident_kernel<0" \
        --fetch <FETCH_SIZE counter_collection.csv> --write <WRITE_SIZE counter_collection.csv>

--kernel may be repeated for a record that covers a whole call (the prefill record: the
split, the two GEMM kernels and the combine): the kernels' means are then summed.

Both counters are in KiB per dispatch.  Each is scaled by what it reads for the
calibration copy (a kernel that reads and writes a known number of bytes): on this
device FETCH_SIZE counts half of what a copy reads.  The record names the digest of the
kernel sources it was measured on; bench.py reports null once they change.
"""
from __future__ import annotations

import argparse
import csv
import json
import statistics
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
COPY_BYTES = 512 << 20  # what bench.py --copy-calibration moves each way per dispatch


def counter_values(path: str, counter: str, kernel_substring: str) -> list[float]:
    with open(path, newline="") as fh:
        return [float(row["Counter_Value"]) for row in csv.DictReader(fh)
                if row["Counter_Name"] == counter and kernel_substring in row["Kernel_Name"]]


def copy_scale(path: str, counter: str) -> tuple[float, float]:
    """(factor, raw KiB of the calibration copy): the copy is the dispatch whose reading is
    nearest to its known size or to half of it."""
    with open(path, newline="") as fh:
        rows = [(float(r["Counter_Value"]), r["Kernel_Name"]) for r in csv.DictReader(fh)
                if r["Counter_Name"] == counter]
    want = COPY_BYTES / 1024.0
    near = [v for v, name in rows if ("copy" in name.lower() or "elementwise" in name.lower())
            and any(abs(v - want / d) <= 0.02 * want / d for d in (1.0, 2.0))]
    if not near:
        raise SystemExit(f"{path}: no dispatch reads like the {COPY_BYTES >> 20} MiB calibration copy")
    raw = statistics.median(near)
    return want / raw, raw


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", required=True)
    ap.add_argument("--kernel", required=True, action="append",
                    help="substring of the dominant kernel's name; given several times, the kernels of "
                         "one call (each launched once per call): their per-dispatch means are summed")
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--out", default=str(ROOT / "profiles" / "traffic.json"))
    args = ap.parse_args()
    sys.path.insert(0, str(ROOT))
    import bench

    f_scale, f_copy = copy_scale(args.fetch, "FETCH_SIZE")
    w_scale, w_copy = copy_scale(args.write, "WRITE_SIZE")
    fetch_kib = write_kib = 0.0
    for name in args.kernel:
        fetch = counter_values(args.fetch, "FETCH_SIZE", name)
        write = counter_values(args.write, "WRITE_SIZE", name)
        if not fetch or not write:
            raise SystemExit(f"no dispatch of a kernel named *{name}* in the counter files")
        fetch_kib += statistics.mean(fetch)
        write_kib += statistics.mean(write)
    read_bytes = fetch_kib * 1024.0 * f_scale
    write_bytes = write_kib * 1024.0 * w_scale
    out = Path(args.out)
    table = json.loads(out.read_text()) if out.is_file() else {}
    table[args.workload] = {
        "kernel": args.kernel[0] if len(args.kernel) == 1 else args.kernel,
        "traffic_bytes": round(read_bytes + write_bytes),
        "read_bytes": round(read_bytes),
        "write_bytes": round(write_bytes),
        "fetch_size_kib_raw": round(fetch_kib, 1),
        "write_size_kib_raw": round(write_kib, 1),
        "fetch_scale": round(f_scale, 4),
        "write_scale": round(w_scale, 4),
        "copy_fetch_kib_raw": round(f_copy, 1),
        "copy_write_kib_raw": round(w_copy, 1),
        "dispatches": [len(fetch), len(write)],
        "sources_sha16": bench.sources_digest(),
    }
    out.write_text(json.dumps(table, indent=1, sort_keys=True) + "\n")
    print(json.dumps(table[args.workload]))


if __name__ == "__main__":
    main()
