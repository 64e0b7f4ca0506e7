"""HBM traffic per batch from two rocprofv3 counter runs of bench.py, as a small record that bench.py reads.

  python -m mako_amd.traffic_record --workload config3 --fetch DIR --write DIR --copy-mb 256 --out profiles/NAME.json

DIR: the output directories of `rocprofv3 --pmc FETCH_SIZE` and `rocprofv3 --pmc WRITE_SIZE` runs (csv output) of
`bench.py --workload W --calibrate-copy-mb N`.  Each counter is scaled by what it reads for that run's one device-to-
device copy of N MiB (a kernel of known traffic: N MiB read, N MiB written).  The record carries a digest of the
kernel sources it was measured on; bench.py reports the figure only while the sources still hash to it.
"""
import argparse
import csv
import glob
import hashlib
import json
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
KERNELS = ("scan_kernel", "finish_kernel", "plan_kernel", "sort_kernel", "tail_kernel")


def kernel_sources_digest():
    """sha256 over the HIP sources and headers the library is built from (names and contents, sorted)."""
    h = hashlib.sha256()
    names = sorted(glob.glob(os.path.join(HERE, "csrc", "*.h")) + glob.glob(os.path.join(HERE, "csrc", "*.hip"))
                   + [os.path.join(ROOT, "include", "mako_sampler.h")])
    for n in names:
        h.update(os.path.basename(n).encode() + b"\0")
        with open(n, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()


def load_record(path, workload):
    """The record's traffic figure (bytes per batch) if it was measured on the sources as they are now, else None."""
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("workload") != workload or rec.get("kernel_sources_sha256") != kernel_sources_digest():
        return None
    return rec.get("traffic_bytes_per_batch")


def _per_kernel(directory, counter):
    """{kernel family: (dispatches, mean counter value)}, and the copy kernel's mean, from a counter_collection csv."""
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit("no *counter_collection.csv under " + directory)
    acc, copy = {}, []
    for path in files:
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                name, v = row["Kernel_Name"], float(row["Counter_Value"])
                if "copyBuffer" in name:
                    copy.append(v)
                for k in KERNELS:
                    if k in name:
                        acc.setdefault(k, []).append(v)
    if not copy:
        raise SystemExit("no device-to-device copy dispatch in %s: run bench.py with --calibrate-copy-mb" % directory)
    return {k: (len(v), sum(v) / len(v)) for k, v in acc.items()}, max(copy)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", required=True)
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--copy-mb", type=int, required=True)
    ap.add_argument("--algorithmic-bytes", type=float, default=None)
    ap.add_argument("--out", required=True)
    a = ap.parse_args()
    copy_kib = a.copy_mb * 1024.0
    fetch, fetch_copy = _per_kernel(a.fetch, "FETCH_SIZE")
    write, write_copy = _per_kernel(a.write, "WRITE_SIZE")
    f_scale, w_scale = copy_kib / fetch_copy, copy_kib / write_copy
    kernels = {}
    # a batch = one dispatch of every kernel that ran; a kernel the batch skipped has no dispatches
    batches = max(n for n, _ in fetch.values())
    fetched = written = 0.0
    for k in KERNELS:
        if k not in fetch:
            continue
        nf, vf = fetch[k]
        nw, vw = write.get(k, (0, 0.0))
        kib_f, kib_w = vf * f_scale * nf / batches, vw * w_scale * nw / batches
        kernels[k] = dict(fetch_kib_per_batch=round(kib_f, 1), write_kib_per_batch=round(kib_w, 1))
        fetched += kib_f
        written += kib_w
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "HEAD"], capture_output=True, text=True,
                                check=True).stdout.strip()
        dirty = bool(subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "mako_amd/csrc", "include"],
                                    capture_output=True, text=True, check=True).stdout.strip())
    except (OSError, subprocess.CalledProcessError):
        commit, dirty = None, None
    rec = dict(workload=a.workload, commit=commit, commit_tree_dirty=dirty,
               kernel_sources_sha256=kernel_sources_digest(),
               counters="rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE, KiB per dispatch, one run each",
               calibration=dict(copy_kib=copy_kib, fetch_counter_for_copy=fetch_copy, write_counter_for_copy=write_copy,
                                fetch_scale=f_scale, write_scale=w_scale),
               batches=batches, kernels=kernels,
               fetch_bytes_per_batch=fetched * 1024.0, write_bytes_per_batch=written * 1024.0,
               traffic_bytes_per_batch=(fetched + written) * 1024.0)
    if a.algorithmic_bytes:
        rec["algorithmic_bytes_per_batch"] = a.algorithmic_bytes
        rec["traffic_over_algorithmic"] = rec["traffic_bytes_per_batch"] / a.algorithmic_bytes
    with open(a.out, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
