#!/usr/bin/env python3
"""Compare two raw output files; prints the three blocks of the reference's
examples/data_diff.py:8-25 (absolute diff min/max/mean, relative diff with the
``+1e-10`` denominator, and the count of elements whose absolute diff exceeds
1 ... 1e-7).  ``data_diff`` also returns the numbers for programmatic use."""
from __future__ import annotations

import argparse

import numpy as np

BOUNDS = [1, 1e-1, 1e-2, 1e-3, 1e-4, 1e-5, 1e-6, 1e-7]


def diff_stats(data0: np.ndarray, data1: np.ndarray):
    data0 = data0.astype(np.float32)
    data1 = data1.astype(np.float32)
    abs_diff = np.abs(data0 - data1)
    rel_diff = np.abs(data0 - data1) / (np.abs(data0) + 1e-10)
    return {
        "abs": (float(np.min(abs_diff)), float(np.max(abs_diff)), float(np.mean(abs_diff))),
        "rel": (float(np.min(rel_diff)), float(np.max(rel_diff)), float(np.mean(rel_diff))),
        "bounds": {b: int(np.count_nonzero(abs_diff > b)) for b in BOUNDS},
    }


def data_diff(standard: str, compare: str, type: str = "f32"):
    dtype = {"f32": np.float32, "f16": np.float16}[type]
    stats = diff_stats(np.fromfile(standard, dtype=dtype), np.fromfile(compare, dtype=dtype))
    a, r = stats["abs"], stats["rel"]
    print(f"Absolute diff:\tMin:{a[0]}\tMax:{a[1]}\tMean:{a[2]}")
    print(f"Relative diff:\tMin:{r[0]}\tMax:{r[1]}\tMean:{r[2]}")
    for bound, num in stats["bounds"].items():
        print(f"Bound {bound}:\t{num}")
    return stats


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("standard", type=str, help="Standard Data")
    ap.add_argument("compare", type=str, help="Compare Data")
    ap.add_argument("--type", type=str, default="f32")
    a = ap.parse_args()
    data_diff(a.standard, a.compare, a.type)


if __name__ == "__main__":
    main()
