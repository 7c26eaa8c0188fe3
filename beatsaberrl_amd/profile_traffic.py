"""HBM traffic of the fused forward from rocprofv3 counters -> a small JSON that bench.py reports.

    python -m beatsaberrl_amd.profile_traffic COUNTER_DIR --out profiles/<name>.json

COUNTER_DIR holds four `rocprofv3 --pmc <counter> --output-format csv` runs, one per
sub-directory:
    copy_FETCH_SIZE, copy_WRITE_SIZE   python3 bench.py --calib-copy 256
    fwd_FETCH_SIZE,  fwd_WRITE_SIZE    python3 bench.py --no-cpu --no-eager --steps 5 --warmup 2
FETCH_SIZE and WRITE_SIZE are KiB per dispatch in the counter's own unit; the copy runs
(256 MiB read, 256 MiB written per dispatch) give the factor from that unit to bytes.
The JSON carries a hash of the kernel sources, and `load_if_current` hands the figure out
only while the sources still hash the same - a rebuilt kernel reports no traffic until
the counters are taken again.

The reference has no counterpart (its audits note that hardware counters were unavailable
on its pods, PERF_AUDIT_2026-08-16.md:22-25)."""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import hashlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_SOURCES = ("csrc/cfg_forward.hip", "csrc/bsrl_common.h")
FORWARD_KERNELS = ("cfg_pair_kernel", "cfg_forward_kernel")


def sources_sha256() -> str:
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(HERE, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _per_kernel(counter_dir, tag):
    """kernel name -> average counter value per dispatch (dispatches of one name are averaged)."""
    files = glob.glob(os.path.join(counter_dir, tag, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise SystemExit(f"no counter_collection.csv under {counter_dir}/{tag}")
    agg = collections.defaultdict(list)
    with open(files[0]) as f:
        for row in csv.DictReader(f):
            agg[row["Kernel_Name"]].append(float(row["Counter_Value"]))
    return {k: (sum(v) / len(v), len(v)) for k, v in agg.items()}


def summarise(counter_dir, copy_mib=256):
    out = {"kernel_sources_sha256": sources_sha256(), "kernel_sources": list(KERNEL_SOURCES), "kernels": {},
           "calibration": {}}
    total = 0.0
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        copies = _per_kernel(counter_dir, "copy_" + counter)
        # the calibration run's copies: the kernel dispatched 5 times (the fill of the source buffer runs once)
        cname, (cval, cn) = max(((k, v) for k, v in copies.items() if v[1] == 5), key=lambda kv: kv[1][0])
        factor = copy_mib * 1024.0 / cval                 # KiB moved per KiB the counter reads
        out["calibration"][counter] = {"copy_kernel": cname[:60], "reading_kib": round(cval, 1), "dispatches": cn,
                                       "true_kib": copy_mib * 1024, "factor": round(factor, 4)}
        for name, (val, n) in _per_kernel(counter_dir, "fwd_" + counter).items():
            if not any(k in name for k in FORWARD_KERNELS):
                continue
            # the HEAD and TAIL launches are two instantiations of one template: keep them apart by their arguments
            key = name if len(name) < 120 else name[:120]
            k = out["kernels"].setdefault(key, {})
            k[counter + "_reading_kib"] = round(val, 1)
            k[counter + "_bytes"] = int(val * factor * 1024)
            k["dispatches"] = n
            total += val * factor * 1024
    out["hbm_bytes_per_forward"] = int(total)
    return out


def load_if_current(path):
    """HBM bytes per forward from a summary written by this module, or None when the file is missing or was taken on
    other kernel sources."""
    try:
        with open(path) as f:
            d = json.load(f)
    except (OSError, ValueError):
        return None
    if d.get("kernel_sources_sha256") != sources_sha256():
        return None
    return d.get("hbm_bytes_per_forward")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("counter_dir")
    ap.add_argument("--out", required=True)
    ap.add_argument("--copy-mib", type=int, default=256)
    ap.add_argument("--command", default="", help="the command line that produced counter_dir, recorded in the summary")
    a = ap.parse_args()
    s = summarise(a.counter_dir, a.copy_mib)
    s["command"] = a.command
    with open(a.out, "w") as f:
        json.dump(s, f, indent=1)
        f.write("\n")
    print(json.dumps({k: s[k] for k in ("hbm_bytes_per_forward", "calibration")}))


if __name__ == "__main__":
    main()
