#!/usr/bin/env python3
"""Writes tests/golden/add_ref_3x640x640_sample.npz.

Runs the reference's own compiled add model (examples/add.ll, built into
oracle/_ref/libadd_ref.so by oracle/Makefile: only possible where the
reference checkout is present) on seeded (3,640,640) fp32 inputs and keeps a
fixed sample of positions: input bits and output bits.  The first 64 sampled
positions are overwritten with IEEE special values (NaN, +-Inf, +-0, denormals,
cancelling pairs, values that round) before the run, so the fixture also pins
the add's behaviour on them.

    python tests/golden/make_add_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

SEED = 20240
N_SAMPLE = 4096


def specials():
    f = np.float32
    tiny = np.float32(1e-45)  # smallest denormal
    vals = [
        (f("nan"), f(1.0)), (f(1.0), f("nan")), (f("inf"), f(1.0)), (f("-inf"), f(1.0)),
        (f("inf"), f("-inf")), (f("inf"), f("inf")), (f(0.0), f(-0.0)), (f(-0.0), f(-0.0)),
        (f(0.0), f(0.0)), (tiny, tiny), (tiny, -tiny), (f(1.17549435e-38), -tiny),
        (f(1.17549421e-38), f(1.17549421e-38)), (f(3.4028235e38), f(3.4028235e38)),
        (f(3.4028235e38), f(1e31)), (f(-3.4028235e38), f(-3.4028235e38)),
        (f(1.0), f(5.9604645e-08)), (f(1.0), f(5.96046519e-08)), (f(1.0), f(1.7881393e-07)),
        (f(16777216.0), f(1.0)), (f(16777216.0), f(3.0)), (f(0.1), f(0.2)), (f(1e-20), f(-1e-20)),
        (f(0.3), f(-0.1)), (f(123456.789), f(-123456.7)), (f(1.5), f(-1.5)),
    ]
    a = np.array([v[0] for v in vals], np.float32)
    b = np.array([v[1] for v in vals], np.float32)
    return a, b


def main():
    if not oracle.ref_add_available():
        raise SystemExit("oracle/_ref/libadd_ref.so is not built (needs /root/reference): run make -C oracle")
    rng = np.random.Generator(np.random.PCG64(SEED))
    a = rng.uniform(-1.0, 1.0, (3, 640, 640)).astype(np.float32)
    b = rng.uniform(-1.0, 1.0, (3, 640, 640)).astype(np.float32)
    idx = np.sort(rng.choice(a.size, N_SAMPLE, replace=False)).astype(np.int64)
    sa, sb = specials()
    a.reshape(-1)[idx[: sa.size]] = sa
    b.reshape(-1)[idx[: sb.size]] = sb
    c = oracle.ref_add_3x640x640(a, b)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "add_ref_3x640x640_sample.npz")
    np.savez_compressed(out, seed=np.int64(SEED), idx=idx, n_special=np.int64(sa.size),
                        a_bits=a.reshape(-1)[idx].view(np.uint32),
                        b_bits=b.reshape(-1)[idx].view(np.uint32),
                        c_bits=c.reshape(-1)[idx].view(np.uint32),
                        c_xor_checksum=np.bitwise_xor.reduce(c.reshape(-1).view(np.uint32)),
                        c_sum_checksum=np.uint64(c.reshape(-1).view(np.uint32).astype(np.uint64).sum()))
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
