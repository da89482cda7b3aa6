#!/usr/bin/env python3
"""Turns two rocprofv3 counter passes over bench.py into profiles/hbm_traffic.json,
the file bench.py reads its `roofline.traffic` figures from.

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/fetch -o p -- python3 bench.py --no-cpu --no-ceilings --copy-calibration --steps 50 --repeats 1
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/write -o p -- python3 bench.py --no-cpu --no-ceilings --copy-calibration --steps 50 --repeats 1
    python3 multi-device-model-compiler_amd/tools/pmc_traffic.py OUT/fetch OUT/write --commit $(git rev-parse --short HEAD) -o profiles/hbm_traffic.json

FETCH_SIZE and WRITE_SIZE count KiB per dispatch in units that depend on the
request size; both are scaled by what the same counter reads for the 64 MiB
device copies of --copy-calibration (64 MiB fetched, 64 MiB written), so the
result is in bytes.  A dispatch is assigned to a bench entry by kernel name and
grid size (threads); dispatches that match nothing are listed on stderr.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import re
import sys

COPY_BYTES = 64 << 20

# (the profiler prints some names demangled and some not: both spellings are matched)
def fmha(d, causal):
    c = "true" if causal else "false"
    return rf"fmha_fwd_kernel(<_Float16, ?{d}, ?\d+, ?{c}|IDF16_Li{d}ELi\d+ELb{int(causal)}E)"


# the plain LayerNorm (template argument RESIDUAL = false), not the add-residual form the layers launch
LN_F32 = r"layernorm_rows_kernel(<float, ?\d+, ?\d+, ?false|IfLi\d+ELi\d+ELb0E)"
LN_F16 = r"layernorm_rows_kernel(<_Float16, ?\d+, ?\d+, ?false|IDF16_Li\d+ELi\d+ELb0E)"

# bench entry -> (regex on the kernel name, grid size in threads or None for any, algorithmic bytes)
ENTRIES = {
    "layernorm_f32": (LN_F32, 4096 * 64, 25_171_968),
    "layernorm_f16": (LN_F16, 4096 * 32, 12_585_984),
    "add_f32": (r"add_f32_vec4_kernel", 1200 * 256, 14_745_600),
    "layernorm_f32_large": (LN_F32, 262144 * 64, 1_610_618_880),
    "add_f32_large": (r"add_f32_vec4_kernel", (1 << 28) // 4, 3_221_225_472),
    "fmha_b32_s128": (fmha(64, False), 32 * 12 * 1 * 256, 25_165_824),
    "fmha_b8_s512_masked": (fmha(64, False), 8 * 16 * 4 * 256, 33_554_464),
    "fmha_b32_s512": (fmha(64, False), 32 * 12 * 4 * 256, 100_663_296),
    "fmha_b32_s512_causal": (fmha(64, True), None, 100_663_296),
    "fmha_d128_b32_s512": (fmha(128, False), 32 * 8 * 4 * 256, 134_217_728),
    "fmha_d128_b4_s2048": (fmha(128, False), 4 * 32 * 16 * 256, 268_435_456),
    "fmha_b4_s4096": (fmha(64, False), 4 * 16 * 16 * 256, 134_217_728),       # blocks of 256 queries
    "fmha_d256_b4_s2048": (fmha(256, False), 4 * 8 * 16 * 256, 134_217_728),
}
COPY_KERNEL = r"copyBuffer"


def read_pass(folder: str, counter: str):
    """{(kernel name, grid size): [value per dispatch]} for one counter."""
    files = glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        sys.exit(f"no *counter_collection.csv under {folder}")
    per = collections.defaultdict(list)
    for path in files:
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                per[(row["Kernel_Name"], int(row["Grid_Size"]))].append(float(row["Counter_Value"]))
    return per


def mean(v):
    return sum(v) / len(v)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("fetch_dir")
    ap.add_argument("write_dir")
    ap.add_argument("--commit", required=True, help="commit the measured kernels were built from")
    ap.add_argument("-o", "--output", default="profiles/hbm_traffic.json")
    args = ap.parse_args()
    fetch, write = read_pass(args.fetch_dir, "FETCH_SIZE"), read_pass(args.write_dir, "WRITE_SIZE")

    def copy_value(per):
        vals = [mean(v) for (name, _grid), v in per.items() if re.search(COPY_KERNEL, name) and mean(v) > 1000]
        if not vals:
            sys.exit("no calibration copy in the pass: run bench.py with --copy-calibration")
        return max(vals)

    fscale = COPY_BYTES / copy_value(fetch)  # bytes per counter unit
    wscale = COPY_BYTES / copy_value(write)
    out = {"commit": args.commit,
           "method": "rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE over bench.py --copy-calibration, means per dispatch, "
                     "each scaled by the same counter's reading for a 64 MiB device copy",
           "bytes_per_unit": {"FETCH_SIZE": round(fscale, 2), "WRITE_SIZE": round(wscale, 2)}, "kernels": {}}
    used = set()
    for entry, (pattern, grid, algorithmic) in ENTRIES.items():
        keys = [k for k in fetch if re.search(pattern, k[0]) and (grid is None or k[1] == grid)]
        if not keys or not all(k in write for k in keys):
            print(f"[pmc_traffic] no dispatch for {entry}", file=sys.stderr)
            continue
        f = mean([x for k in keys for x in fetch[k]])
        w = mean([x for k in keys for x in write[k]])
        used.update(keys)
        total = f * fscale + w * wscale
        out["kernels"][entry] = {"kernel": keys[0][0][:120], "grid_threads": keys[0][1], "dispatches": sum(len(fetch[k]) for k in keys),
                                 "fetch_units": round(f, 1), "write_units": round(w, 1), "bytes": int(round(total, -3)),
                                 "algorithmic_bytes": algorithmic, "ratio": round(total / algorithmic, 4)}
    for k in fetch:
        if k not in used and not re.search(COPY_KERNEL, k[0]):
            print(f"[pmc_traffic] unassigned: grid {k[1]:>10} x{len(fetch[k]):<4} {k[0][:100]}", file=sys.stderr)
    with open(args.output, "w") as fh:
        json.dump(out, fh, indent=1)
        fh.write("\n")
    print(json.dumps(out["kernels"], indent=1))


if __name__ == "__main__":
    main()
