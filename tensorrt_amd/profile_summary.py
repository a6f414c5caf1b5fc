"""Turns the raw rocprofv3 output of the profile commands into the figures bench.py and profiles/ quote.

    python -m tensorrt_amd.profile_summary --workload encoder \\
        --stats out/enc_stats/bench_kernel_stats.csv \\
        --fetch out/enc_fetch/bench_counter_collection.csv \\
        --write out/enc_write/bench_counter_collection.csv [--update profiles/traffic.json]

The FETCH_SIZE / WRITE_SIZE runs must have been made with bench.py's --pmc-calibration, whose plain copy of known
size (256 MiB read, 256 MiB written) is the yardstick the counter readings are scaled by.  Prints the per-kernel
durations and traffic; with --update, writes the HBM-side bytes per launch of the kernels bench.py reports under the
workload's key of that JSON file, which bench.py reads for its `traffic` fields.
"""
from __future__ import annotations

import argparse
import collections
import csv
import json
import re

CALIBRATION_KIB = 256 * 1024
# bench.py's kernel keys -> a pattern of the kernel's (demangled) name, per workload
KERNELS = {
    "encoder": {"ffn1_gemm_gelu": r"int8_linear_dma_kernel<\w+,\s*\w+,\s*1\b", "attention": r"fmha_i8_\w*kernel",
                "skipln": r"skipln_interleaved_kernel", "gemm_affine": r"int8_linear_dma_kernel<\w+,\s*\w+,\s*0\b"},
    "layer": {"attention": r"fmha_i8_\w*kernel", "skipln": r"skipln_interleaved_kernel"},
}


def counter_means(path):
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        agg[r["Kernel_Name"]].append(float(r["Counter_Value"]))
    return {k: (sum(v) / len(v), len(v)) for k, v in agg.items()}


def calibration(means):
    """The elementwise copy of the calibration leg: torch's `add(src, 1, out=dst)` on signed bytes."""
    cands = [(v[0], k) for k, v in means.items() if "elementwise" in k and "add<signed char>" in k]
    if not cands:
        raise SystemExit("no calibration copy in the counter file: run bench.py with --pmc-calibration")
    return max(cands)[0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", choices=sorted(KERNELS), required=True)
    ap.add_argument("--stats")
    ap.add_argument("--fetch", required=True)
    ap.add_argument("--write", required=True)
    ap.add_argument("--update", help="JSON file whose entry for this workload is replaced")
    args = ap.parse_args()

    if args.stats:
        print("kernel | calls | average ns | min ns | max ns | share")
        for r in list(csv.DictReader(open(args.stats)))[:12]:
            print(f"{r['Name'][:100]} | {r['Calls']} | {r['AverageNs']} | {r['MinNs']} | {r['MaxNs']} | {r['Percentage']}")
    fetch, write = counter_means(args.fetch), counter_means(args.write)
    f_cal, w_cal = calibration(fetch), calibration(write)
    fs, ws = CALIBRATION_KIB / f_cal, CALIBRATION_KIB / w_cal
    print(f"calibration copy: FETCH_SIZE {f_cal:.0f} -> x{fs:.3f}, WRITE_SIZE {w_cal:.0f} -> x{ws:.3f} (KiB)")
    entry = {"fetch_scale": round(fs, 4), "write_scale": round(ws, 4), "kernels": {}}
    for key, pat in KERNELS[args.workload].items():
        f = [(v, k) for k, v in fetch.items() if re.search(pat, k)]
        w = [(v, k) for k, v in write.items() if re.search(pat, k)]
        if not f or not w:
            continue
        (fv, fn), name = max(f, key=lambda t: t[0][1])       # the instantiation with the most launches
        (wv, wn) = dict((k, v) for v, k in w)[name]
        fetched, written = fv * fs * 1024, wv * ws * 1024
        entry["kernels"][key] = {"kernel": name[:120], "FETCH_SIZE": round(fv), "WRITE_SIZE": round(wv),
                                 "fetched_bytes": round(fetched), "written_bytes": round(written),
                                 "traffic_bytes": round(fetched + written), "launches": fn}
        print(f"{key}: FETCH_SIZE {fv:.0f} = {fetched / 1e6:.1f} MB, WRITE_SIZE {wv:.0f} = {written / 1e6:.1f} MB, "
              f"total {(fetched + written) / 1e6:.1f} MB per launch ({fn} launches)  [{name[:80]}]")
    if args.update:
        try:
            doc = json.load(open(args.update))
        except FileNotFoundError:
            doc = {}
        doc[args.workload] = entry
        json.dump(doc, open(args.update, "w"), indent=1, sort_keys=True)
        print("updated", args.update)


if __name__ == "__main__":
    main()
