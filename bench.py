#!/usr/bin/env python3
"""Benchmark of the device kernel library on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input, with
all inputs already resident in HBM when the timed region starts.  The headline
workload is the LayerNorm configuration of the benchmark definition (configs[1]:
fp32 (32,128,768), eps 1e-5); the other configurations (add, fp16 LayerNorm,
fused MHA at three shapes, the BERT-base layer) are measured in the same run
and reported under "kernels" in the same JSON line, each against the roofline
that bounds it.

Timing: K launches are enqueued back to back on one stream between two HIP
events recorded on that same stream.  The calls are made from a C++ loop
(lib/libmgpu_bench_loops.so, K calls of the same C-ABI entry point a compiled
model calls) because a ctypes call costs more host time than a streaming
kernel runs; --graph times a hipGraph of K ctypes launches instead and gives
the same figures within a few per cent.  Memory-bound kernels rotate
through enough distinct buffer sets (> 256 MiB in total) that no launch finds
its operands in the Infinity Cache left by an earlier one; the cache-resident
("warm") figure is reported next to it.

Every figure is the median of --repeats timed regions.  The headline's region is
the contract's: --warmup untimed launches, then exactly --steps timed ones.  The
other entries keep at least the default region (200 launches behind 20 untimed
ones, fractions of it for the long kernels) whatever --steps asked for: twenty
launches of a 4 us kernel are mostly the start of the queue, and twenty of a
matrix kernel end before the device has settled into its clocks.

The CPU baseline follows the reference's CPU runner
(tools/multi-device-cpu-runner/multi-device-cpu-runner.cpp:65-82: a clock
around each rerun, the mean over the reruns) on this build's CPU op library
(lib/libmcpu_ops.so, plain C++ / OpenMP, fp32 arithmetic), at one thread and
at all host cores, on a bounded number of reruns; the reference's own compiled
add model (oracle/_ref/libadd_ref.so, single threaded) is timed beside it when
it has been built.  It is a reported baseline, not the target.

"ceilings" reports what the device gives the simplest kernel of each kind in
the same run: a 1 GiB copy, a copy at the headline's grid and byte count, and
a register-fed MFMA loop with the shader clock read in the kernel.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
MALL_BYTES = 256 << 20
CACHE_MULTIPLE = 2.0  # footprint of the rotating buffer sets in units of the Infinity Cache (--cache-multiple)
# HBM bytes per launch as counted by the hardware: profiles/hbm_traffic.json is
# written from two rocprofv3 --pmc passes over this script (FETCH_SIZE, then
# WRITE_SIZE, each scaled by what the same counter reads for the 64 MiB copy of
# --copy-calibration) by tools/pmc_traffic.py and names the commit the kernels
# were built from.  A kernel without an entry there reports traffic null.


def load_traffic():
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            data = json.load(f)
        return {k: v.get("bytes") for k, v in data.get("kernels", {}).items()}, data.get("commit")
    except (OSError, ValueError):
        return {}, None


TRAFFIC_BYTES, TRAFFIC_COMMIT = load_traffic()


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=7, help="timed regions of --steps launches each; the median is reported")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the copy / launch-floor / MFMA-loop probes")
    ap.add_argument("--cache-multiple", type=float, default=2.0,
                    help="total footprint of the rotating buffer sets of the cold measurements, in units of the 256 MiB "
                         "Infinity Cache")
    ap.add_argument("--no-runner", action="store_true", help="skip the end-to-end --rerun figures of the two runners")
    ap.add_argument("--no-sdpa", action="store_true",
                    help="skip timing torch's scaled_dot_product_attention beside the attention entries")
    ap.add_argument("--no-torch-ref", action="store_true",
                    help="skip timing torch's own layer_norm / add / layer composition beside the entries")
    ap.add_argument("--tune-gemm", action="store_true",
                    help="measure the four GEMM shapes of the BERT-base layer with the tuner of the launch-loop library (library candidates "
                         "against the hand-written kernel) and print the lines of csrc/kernels/gemm_table.inc on stderr")
    ap.add_argument("--fmha-phases", action="store_true",
                    help="also run the attention kernel's profiling entry point at b32 s512 h12 d64 and report where a "
                         "block's time goes (prologue, tiles, epilogue) from the kernel's own clocks")
    ap.add_argument("--graph", action="store_true",
                    help="time a hipGraph of K ctypes launches instead of the C++ launch loops")
    ap.add_argument("--no-graph", action="store_true", help="with --graph: enqueue the ctypes launches directly")
    ap.add_argument("--only", type=str, default="", help="comma list of kernels to run besides the headline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run plain device copies of 64 MiB (for scaling FETCH_SIZE / WRITE_SIZE counters)")
    return ap.parse_args()


class Timer:
    """Times `steps` launches of fn(i) on the current torch stream."""

    def __init__(self, torch, use_graph: bool):
        self.torch = torch
        self.use_graph = use_graph

    def run(self, fn, steps: int, warmup: int, repeats: int = 1) -> float:
        """Median over `repeats` timed regions of the milliseconds for exactly `steps` launches."""
        return float(np.median([self.run_once(fn, steps, warmup) for _ in range(max(1, repeats))]))

    def run_once(self, fn, steps: int, warmup: int) -> float:
        torch = self.torch
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for i in range(warmup):
                fn(i)
            stream.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            graph = None
            if self.use_graph:
                try:
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=stream):
                        for i in range(steps):
                            fn(i)
                    graph.replay()  # untimed first replay (upload)
                    stream.synchronize()
                except Exception as exc:  # capture unsupported for this op: time direct launches
                    print(f"[bench] graph capture failed ({exc}); timing direct launches", file=sys.stderr)
                    graph = None
                    torch.cuda.synchronize()
            torch.cuda.synchronize()
            e0.record(stream)
            if graph is not None:
                graph.replay()
            else:
                for i in range(steps):
                    fn(i)
            e1.record(stream)
            e1.synchronize()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1)


def device_info(torch) -> dict:
    """What the device reports about itself, with the peaks those figures imply:
    dense fp16 MFMA = CUs x 4 SIMDs x 1024 flop/clock x shader clock, HBM =
    2 transfers/clock x memory clock x bus width.  The roofline objects use the
    published 2.5 PFLOP/s and 8 TB/s; these are printed beside them."""
    pr = torch.cuda.get_device_properties(0)
    cus = getattr(pr, "multi_processor_count", None)
    clk_khz = getattr(pr, "clock_rate", None)
    mclk_khz = getattr(pr, "memory_clock_rate", None)
    bus = getattr(pr, "memory_bus_width", None)
    info = {"arch": getattr(pr, "gcnArchName", None), "compute_units": cus, "shader_clock_mhz": clk_khz and clk_khz / 1e3,
            "memory_clock_mhz": mclk_khz and mclk_khz / 1e3, "memory_bus_bits": bus,
            "hbm_bytes": getattr(pr, "total_memory", None)}
    try:  # torch does not report clocks on this platform; the runtime's own listing does
        import re
        import subprocess
        txt = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=30).stdout
        for agent in txt.split("*******")[1:]:
            if "gfx950" in agent and "Max Clock Freq. (MHz)" in agent:
                mhz = float(re.search(r"Max Clock Freq\. \(MHz\):\s*(\d+)", agent).group(1))
                info["shader_clock_mhz"] = info["shader_clock_mhz"] or mhz
                clk_khz = clk_khz or mhz * 1e3
                break
    except Exception:
        pass
    if cus and clk_khz:
        info["mfma_f16_peak_tflops_at_reported_clock"] = round(cus * 4 * 1024 * clk_khz * 1e3 / 1e12, 1)
    if mclk_khz and bus:
        info["hbm_peak_gbs_at_reported_clock"] = round(2 * mclk_khz * 1e3 * bus / 8 / 1e9, 1)
    return info


def rotating_sets(bytes_per_set: int) -> int:
    """Number of buffer sets (bytes read + bytes written per launch each) whose total footprint is at
    least twice the Infinity Cache: the launch loops walk them round robin without ever restarting, so
    between two uses of a set the device moves a full rotation of other bytes."""
    return max(3, int(CACHE_MULTIPLE * MALL_BYTES + bytes_per_set - 1) // bytes_per_set + 1)


def hbm_entry(name, workload, dtype, bytes_per_launch, ms, steps, warm_ms=None, copy_us=None, copy_what=None):
    """copy_us: microseconds per launch of the plain copy probe with the same bytes in and out (same number
    of input streams, same rotation of buffer sets), timed in the same process right after the kernel."""
    us = ms * 1e3 / steps
    gbs = bytes_per_launch / us / 1e3
    e = {"name": name, "workload": workload, "dtype": dtype, "metric": "GB/s", "value": round(gbs, 1),
         "us_per_launch": round(us, 3),
         "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                      "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES.get(name)},
         "algorithmic_bytes": bytes_per_launch}
    if copy_us:
        e["copy_ceiling"] = {"us_per_launch": round(copy_us, 3), "GB/s": round(bytes_per_launch / copy_us / 1e3, 1),
                             "what": copy_what}
        e["copy_ceiling_GBs"] = e["copy_ceiling"]["GB/s"]
        e["frac_of_copy_ceiling"] = round(copy_us / us, 4)
    if warm_ms is not None:
        wus = warm_ms * 1e3 / steps
        e["cache_resident"] = {"us_per_launch": round(wus, 3), "GB/s": round(bytes_per_launch / wus / 1e3, 1)}
    return e



def cpu_model_name() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baselines(pkg, m, n, ln_bytes) -> dict:
    """Times the CPU op library the way the reference's CPU runner times a model
    (multi-device-cpu-runner.cpp:65-82: one untimed run, then a clock around
    each rerun, mean over the reruns), at one thread and at all host cores, for
    add, LayerNorm fp32, attention b32 s128 and the BERT-base layer.  The number
    of reruns is bounded by time so the whole leg stays near 25 s."""
    lib = ctypes.CDLL(os.path.join(pkg.LIB_DIR, "libmcpu_ops.so"))
    lib.mcpuGetNumThreads.restype = ctypes.c_int32
    all_threads = min(int(lib.mcpuGetNumThreads()), len(os.sched_getaffinity(0)))
    model = cpu_model_name()
    rng = np.random.default_rng(20241)
    P = lambda a: a.ctypes.data_as(ctypes.c_void_p)

    def reruns(fn, budget_s, max_runs):
        fn()  # the model's first run, untimed like the runner's
        times = []
        t_end = time.perf_counter() + budget_s
        while len(times) < max_runs and (len(times) < 2 or time.perf_counter() < t_end):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sum(times) / len(times), len(times)

    def both(fn, budget_s, max_runs, to_value, unit, what):
        res = {}
        for threads in (all_threads, 1):
            lib.mcpuSetNumThreads(threads)
            sec, runs = reruns(fn, budget_s, max_runs)
            res[threads] = (to_value(sec), sec, runs)
        lib.mcpuSetNumThreads(all_threads)
        v, sec, runs = res[all_threads]
        v1, sec1, runs1 = res[1]
        return {"value": round(v, 3), "unit": unit, "cores": all_threads, "threads": all_threads, "cpu_model": model,
                "kind": "port", "seconds_per_run": round(sec, 6),
                "single_thread": {"value": round(v1, 3), "unit": unit, "threads": 1, "seconds_per_run": round(sec1, 6),
                                  "reruns": runs1},
                "sample": f"{what}: mean of {runs} reruns of the entry point of lib/libmcpu_ops.so (fp32 arithmetic, OpenMP) "
                          f"with a clock around each, as multi-device-cpu-runner --rerun does; {runs1} reruns at one thread"}

    out = {}
    x = rng.standard_normal((m, n)).astype(np.float32)
    g = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
    b = (0.02 * rng.standard_normal(n)).astype(np.float32)
    y = np.empty_like(x)
    out["layernorm_f32"] = both(lambda: lib.mcpuLayerNormF32(P(x), P(g), P(b), P(y), ctypes.c_float(1e-5), m, n),
                                1.0, 2000, lambda s: ln_bytes / s / 1e9, "GB/s", f"LayerNorm fp32 ({m},{n})")

    ne = 3 * 640 * 640
    a1 = rng.uniform(-1, 1, ne).astype(np.float32)
    b1 = rng.uniform(-1, 1, ne).astype(np.float32)
    c1 = np.empty_like(a1)
    out["add_f32"] = both(lambda: lib.mcpuAddF32(P(a1), P(b1), P(c1), ctypes.c_int64(ne)), 1.0, 2000,
                          lambda s: 3 * ne * 4 / s / 1e9, "GB/s", "add fp32 (3,640,640)")
    # the reference's own compiled add model (examples/add.ll through llc + gcc, built by
    # oracle/Makefile where the reference checkout exists): single threaded
    import __graft_entry__ as ge
    oracle = ge.load_oracle()
    if oracle.ref_add_available():
        times = oracle.ref_add_seconds(a1.reshape(3, 640, 640), b1.reshape(3, 640, 640), 100)
        sec = sum(times) / len(times)
        out["add_f32"]["reference_model"] = {
            "value": round(3 * ne * 4 / sec / 1e9, 3), "unit": "GB/s", "threads": 1, "cores": 1, "kind": "reference",
            "cpu_model": model, "seconds_per_run": round(sec, 6),
            "sample": f"mean of {len(times)} reruns of _mlir_ciface_main_graph of the reference's examples/add.ll "
                      "(oracle/_ref/libadd_ref.so), the model's malloc of its 4.9 MB output inside the clock as in "
                      "multi-device-cpu-runner"}

    B, S, H, D = 32, 128, 12, 64
    qkv = (rng.standard_normal((B, S, 3, H, D)) / 8).astype(np.float16)
    o = np.empty((B, S, H * D), np.float16)
    flop = 4.0 * B * H * S * S * D
    out["fmha_b32_s128"] = both(lambda: lib.mcpuFusedMHAF16(P(qkv), None, P(o), B, S, H, D, ctypes.c_float(0.125), 0),
                                2.5, 50, lambda s: flop / s / 1e12, "TFLOP/s", "fused MHA fp16 b32 s128 h12 d64")

    d, ffn = 768, 3072
    h16 = lambda *sh: (0.02 * rng.standard_normal(sh)).astype(np.float16)
    gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
    xb = rng.standard_normal((B, S, d)).astype(np.float16)
    W = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d), h16(d), gam(), h16(d)]
    ob = np.empty_like(xb)
    i64 = ctypes.c_int64
    out["bert_layer"] = both(lambda: lib.mcpuBertEncoderLayerF16(P(xb), *[P(w) for w in W], None, P(ob), i64(B), i64(S), i64(d),
                                                                  i64(ffn), i64(H), ctypes.c_float(1e-5)),
                             4.0, 10, lambda s: s * 1e6, "us", "BERT-base encoder layer fp16 (32,128,768)")
    return out


def runner_end_to_end(pkg, reruns: int = 30) -> dict:
    """The reference's own figure (tools/multi-device-gpu-runner/multi-device-gpu-runner.cpp:69-87: the model
    run N times between two events, allocation, host-to-device and device-to-host copies of every run
    included): this build's runners on the device plans of configs[0..2], host buffers pageable as the
    reference's runner allocates them.  PCIe-inclusive, reported beside the kernel-only figures, never as
    `value`."""
    import re
    import subprocess
    import tempfile
    P = os.path.dirname(os.path.abspath(pkg.__file__))
    gpu_runner = os.path.join(P, "bin", "multi-device-gpu-runner")
    cpu_runner = os.path.join(P, "bin", "multi-device-cpu-runner")
    if not (os.path.exists(gpu_runner) and os.path.exists(cpu_runner)):
        return {"error": "runners are not built"}
    rng = np.random.default_rng(20240)
    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        def dat(name, a):
            path = os.path.join(tmp, name)
            a.tofile(path)
            return path
        cases = {
            "add_f32": ("add.plan", [dat("a.dat", rng.uniform(-1, 1, (3, 640, 640)).astype(np.float32)),
                                     dat("b.dat", rng.uniform(-1, 1, (3, 640, 640)).astype(np.float32))], 3 * 4915200),
            "layernorm_f32": ("layernorm.plan", [dat("x.dat", rng.standard_normal((32, 128, 768)).astype(np.float32)),
                                                 dat("g.dat", np.ones(768, np.float32)), dat("be.dat", np.zeros(768, np.float32))],
                              2 * 32 * 128 * 768 * 4),
            "fmha_b32_s128": ("fmha.plan", [dat("qkv.dat", (rng.standard_normal((32, 128, 3, 12, 64)) / 8).astype(np.float16))],
                              32 * 128 * 768 * 2 * 4),
        }
        for name, (plan, files, nbytes) in cases.items():
            entry = {"plan": f"plans/{plan}", "reruns": reruns, "bytes_over_pcie_per_run": nbytes}
            for which, cmd in (("gpu_runner", [gpu_runner, os.path.join(P, "plans", plan), "--ops", os.path.join(pkg.LIB_DIR, "ops.hsaco")]),
                               ("cpu_runner", [cpu_runner, os.path.join(P, "plans", plan)])):
                n = reruns if which == "gpu_runner" or name != "fmha_b32_s128" else 3
                try:
                    r = subprocess.run(cmd + ["--data", ",".join(files), "--rerun", str(n)], capture_output=True, text=True,
                                       timeout=120)
                    m = re.search(r"Average time:\s*([0-9.eE+-]+)\s*seconds", r.stdout)
                    entry[which + "_us_per_run"] = round(float(m.group(1)) * 1e6, 1) if (r.returncode == 0 and m) else None
                except Exception as exc:  # a missing runner or a timeout: say so, the kernel figures stand
                    entry[which + "_us_per_run"] = None
                    entry[which + "_error"] = str(exc)[:200]
            out[name] = entry
    out["what"] = ("multi-device-gpu-runner / multi-device-cpu-runner <plan> --data ... --rerun N: seconds per run of the "
                   "whole model call, device allocation, host-to-device and device-to-host copies included (pageable host "
                   "buffers), as the reference's runner reports it")
    return out


def fmha_phases(torch, lib, loops, dev, gen, B=32, S=512, H=12) -> dict:
    """Per-block clock stamps of the attention kernel (mgpuBenchFusedMHAF16Profile of the launch-loop library):
    how long a block spends before its first tile, per tile, and after its last
    tile, and how the blocks fill the launch."""
    D = 64
    qkv = (torch.randn((B, S, 3, H, D), device=dev, generator=gen) / 8).half()
    out = torch.empty((B, S, H * D), device=dev, dtype=torch.float16)
    nblocks = B * H * ((S + 127) // 128)
    stamps = torch.zeros(nblocks * 10, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        got = loops.mgpuBenchFusedMHAF16Profile(qkv.data_ptr(), out.data_ptr(), B, S, H, D ** -0.5, stamps.data_ptr(), stream)
    torch.cuda.synchronize()
    if got != nblocks:
        raise RuntimeError("mgpuBenchFusedMHAF16Profile failed")
    t = stamps.cpu().numpy().reshape(nblocks, 10).astype(np.float64)
    khz = int(loops.mgpuProbeWallClockKHz()) if loops else 100000
    wall_us = lambda ticks: ticks / khz * 1e3
    k0 = t[:, 4].min()
    start_us, end_us = wall_us(t[:, 4] - k0), wall_us(t[:, 5] - k0)
    total_us = end_us.max()
    ghz = float(np.median((t[:, 3] - t[:, 0]) / np.maximum(1.0, (t[:, 5] - t[:, 4])) * khz / 1e6))
    tiles = (S + 63) // 64
    pro, loop, epi = t[:, 1] - t[:, 0], t[:, 2] - t[:, 1], t[:, 3] - t[:, 2]
    first = start_us < 1.0  # blocks resident from the start of the launch
    q = lambda a: [round(float(np.percentile(a, p)), 1) for p in (10, 50, 90)]
    return {
        "shape": f"b{B} s{S} h{H} d{D}", "blocks": nblocks, "tiles_per_block": tiles,
        "kernel_us_first_entry_to_last_exit": round(float(total_us), 2),
        "shader_clock_ghz": round(ghz, 3),
        "blocks_resident_at_start": int(first.sum()),
        "last_block_entry_us": round(float(start_us.max()), 2),
        "cycles_p10_p50_p90": {
            "prologue_entry_to_first_tile": q(pro), "prologue_of_blocks_resident_at_start": q(pro[first]),
            "prologue_of_later_blocks": q(pro[~first]) if (~first).any() else None,
            "loop_per_tile": q(loop / tiles), "epilogue_last_tile_to_stores_issued": q(epi),
            "per_tile_wait_for_tile_and_barrier": q(t[:, 6] / tiles), "per_tile_score_mfmas": q(t[:, 7] / tiles),
            "per_tile_softmax": q(t[:, 8] / tiles), "per_tile_pv_mfmas": q(t[:, 9] / tiles)},
        "share_of_block_lifetime": {
            "prologue": round(float(pro.sum() / (pro + loop + epi).sum()), 3),
            "tiles": round(float(loop.sum() / (pro + loop + epi).sum()), 3),
            "epilogue": round(float(epi.sum() / (pro + loop + epi).sum()), 3)},
        "block_lifetime_us_p50": round(float(np.median(end_us - start_us)), 2),
        "mfma_cycles_per_tile_per_simd": 3 * 16 * 32,
        "note": "loop_per_tile is one wavefront's time per 64-key tile with 3 wavefronts sharing the SIMD: the SIMD's "
                "matrix pipe needs 3 x 16 x 32 = 1536 cycles for the three tiles that pass in that time",
    }


def measure_ceilings(torch, loops, dev, gen, sp, ptrs, repeats) -> dict:
    """A 1 GiB copy, a copy with the headline's grid and bytes (cold and cache
    resident), and the register-fed MFMA loop at 1-4 wavefronts per SIMD."""
    def med(call):
        t = [call() for _ in range(repeats)]
        return float(np.median(t)) if min(t) >= 0 else None

    res = {}
    big = 1 << 30
    src = torch.empty(big, dtype=torch.uint8, device=dev).random_(generator=gen)
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    ms = med(lambda: loops.mgpuProbeCopy(ptrs([src]), ptrs([dst]), 1, ctypes.c_size_t(big), 10, 2, sp))
    if ms:
        res["copy_1GiB"] = {"GB/s": round(2 * big * 10 / ms / 1e6, 1), "us_per_launch": round(ms * 100, 1),
                            "what": "one 16-byte vector per lane, one block per 256 vectors, 1 GiB read + 1 GiB written"}
    del src, dst
    half = 32 * 128 * 768 * 4  # bytes read (and written) by the headline LayerNorm
    nsets = rotating_sets(2 * half)
    srcs = [torch.empty(half, dtype=torch.uint8, device=dev).random_(generator=gen) for _ in range(nsets)]
    dsts = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(nsets)]
    torch.cuda.synchronize()
    cold = med(lambda: loops.mgpuProbeCopy(ptrs(srcs), ptrs(dsts), nsets, ctypes.c_size_t(half), 100, 10, sp))
    warm = med(lambda: loops.mgpuProbeCopy(ptrs(srcs[:1]), ptrs(dsts[:1]), 1, ctypes.c_size_t(half), 100, 10, sp))
    if cold and warm:
        res["copy_at_headline_size"] = {
            "bytes": 2 * half, "us_per_launch": round(cold * 10, 3), "GB/s": round(2 * half * 100 / cold / 1e6, 1),
            "cache_resident_us_per_launch": round(warm * 10, 3),
            "what": "the same copy kernel at the headline's byte count (12.6 MB in, 12.6 MB out, 3072 blocks): the time "
                    "a launch of that size costs a kernel that does nothing but move the bytes"}
        # the same sets, half of each: the byte count of the fp16 LayerNorm configuration
        quarter = half // 2
        cold16 = med(lambda: loops.mgpuProbeCopy(ptrs(srcs), ptrs(dsts), nsets, ctypes.c_size_t(quarter), 100, 10, sp))
        if cold16:
            res["copy_at_fp16_layernorm_size"] = {
                "bytes": 2 * quarter, "us_per_launch": round(cold16 * 10, 3),
                "GB/s": round(2 * quarter * 100 / cold16 / 1e6, 1),
                "what": "the copy kernel at the byte count of LayerNorm fp16 (32,128,768): 6.3 MB in, 6.3 MB out"}
    del srcs, dsts
    sink = torch.zeros(16, device=dev)
    stamps = torch.zeros(2 * 4096, dtype=torch.int64, device=dev)
    khz = int(loops.mgpuProbeWallClockKHz())
    iters = 4096
    runs = []
    for waves_per_simd in (1, 2, 3, 4):
        blocks = 256 * waves_per_simd
        best = None
        for _ in range(max(3, repeats // 2)):
            sc, cc = ctypes.c_uint64(0), ctypes.c_uint64(0)
            ms = loops.mgpuProbeMfma(ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(stamps.data_ptr()), blocks, iters,
                                     ctypes.byref(sc), ctypes.byref(cc), sp)
            if ms > 0 and (best is None or ms < best[0]):
                best = (ms, sc.value, cc.value)
        if best:
            ms, sc, cc = best
            flop = blocks * 4.0 * iters * 4 * 32 * 32 * 16 * 2
            ghz = sc / cc * khz / 1e6 if cc and khz else None
            runs.append({"wavefronts_per_simd": waves_per_simd, "TFLOP/s": round(flop / ms / 1e9, 1),
                         "shader_clock_ghz_in_kernel": ghz and round(ghz, 3),
                         "clocks_per_mfma": round(sc / (iters * 4.0 * waves_per_simd), 2)})
    if runs:
        res["mfma_f16_loop"] = {"runs": runs, "best_TFLOP/s": max(r["TFLOP/s"] for r in runs),
                                "what": "v_mfma_f32_32x32x16_f16 on four independent accumulators from registers, "
                                        "4096 x 4 per wavefront, every SIMD of the device; shader clock from clock64() "
                                        "against the constant-rate wall_clock64()"}
    # LDS read rate of the attention kernels' operand reads (csrc/tools/bench_probes.hip: probe_lds_read_kernel)
    if hasattr(loops, "mgpuProbeLdsRead"):
        cus = torch.cuda.get_device_properties(dev).multi_processor_count
        lds_iters = 2000
        lds_runs = []
        for mode, name in ((0, "ds_read_b128"), (1, "ds_read_b64_tr_b16"), (2, "ds_read_b64")):
            for waves_per_simd in (2, 3):
                blocks = cus * waves_per_simd
                best = None
                for _ in range(3):
                    sc, cc = ctypes.c_uint64(0), ctypes.c_uint64(0)
                    ms = loops.mgpuProbeLdsRead(ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(stamps.data_ptr()), blocks,
                                                lds_iters, mode, ctypes.byref(sc), ctypes.byref(cc), sp)
                    if ms > 0 and (best is None or ms < best[0]):
                        best = (ms, sc.value, cc.value)
                if best:
                    ms, sc, cc = best
                    nbytes = blocks * 4.0 * lds_iters * 16384
                    ghz = sc / cc * khz / 1e6 if cc and khz else None
                    lds_runs.append({"instruction": name, "wavefronts_per_simd": waves_per_simd,
                                     "TB/s": round(nbytes / ms / 1e9, 1),
                                     "shader_clock_ghz_in_kernel": ghz and round(ghz, 3),
                                     "bytes_per_clock_and_cu": ghz and round(nbytes / ms / 1e6 / cus / ghz, 1)})
        if lds_runs:
            res["lds_read"] = {"runs": lds_runs,
                               "what": "every wavefront re-reads a 16 KiB tile (64 rows of 256 bytes) 2000 times in the "
                                       "operand patterns of the head_dim 128 attention tile: K operands by ds_read_b128, "
                                       "V operands by the transposing ds_read_b64_tr_b16, and plain ds_read_b64; rate from "
                                       "the launch's wall time, per clock with the shader clock read inside the kernel"}
    # the attention tile loop without its bookkeeping (csrc/tools/bench_probes.hip: probe_fmha_loop_kernel)
    kv = (torch.randn((512, 3, 384, 64), device=dev, generator=None) / 8).half()
    stamps = torch.zeros(8 * 256 * 3, dtype=torch.int64, device=dev)
    tiles = 1500
    model = []
    names = {0: "three phases per tile", 1: "half-tile pipeline"}
    for queries, waves_per_simd in ((32, 1), (32, 2), (32, 3), (64, 1), (64, 2)):
        for pipelined in (0, 1):
            for loads in (0, 1):
                variant = pipelined | (2 if queries == 64 else 0) | (4 if loads else 0)
                blocks = 256 * waves_per_simd
                best = None
                for _ in range(2):
                    sc, cc = ctypes.c_double(0), ctypes.c_double(0)
                    ms = loops.mgpuProbeFmhaLoop(ctypes.c_void_p(sink.data_ptr()), ctypes.c_void_p(stamps.data_ptr()),
                                                 ctypes.c_void_p(kv.data_ptr()), blocks, tiles, variant, ctypes.byref(sc),
                                                 ctypes.byref(cc), sp)
                    if ms > 0 and (best is None or ms < best[0]):
                        best = (ms, sc.value, cc.value)
                if not best:
                    continue
                ms, sc, cc = best
                units = queries // 32                      # 32-query blocks per wavefront
                flop = blocks * 4.0 * tiles * units * 16 * 32 * 32 * 16 * 2
                model.append({"queries_per_wavefront": queries, "wavefronts_per_simd": waves_per_simd,
                              "schedule": names[pipelined], "tile_loads_and_barrier": bool(loads),
                              "simd_clocks_per_32_query_tile": round(sc / tiles / waves_per_simd / units, 1),
                              "shader_clock_ghz_in_kernel": round(sc / cc * khz / 1e6, 3) if cc and khz else None,
                              "TFLOP/s": round(flop / ms / 1e9, 1)})
    del kv
    res["fmha_d64_tile_loop_model"] = {
        "runs": model, "mfma_clocks_per_32_query_tile": 16 * 32,
        "what": "the tile loop of the head_dim-64 attention kernel without masks, repair path, prologue and epilogue: per "
                "64-key tile and 32 queries 8 score MFMAs fed by ds_read_b128 of a K tile, the softmax of their results (per "
                "score one fma, one exp2, one add, half a convert), 8 P.V MFMAs fed by the converted scores and "
                "ds_read_b64_tr_b16 of a V tile; in the product kernel's three phases or with every MFMA followed by an "
                "eighth of a half softmax (operand reads three MFMAs ahead); optionally with the product's four "
                "global_load_lds per wavefront and tile and its block barrier; shader clock from clock64() against "
                "wall_clock64(), TFLOP/s from the launch's wall time"}
    return res


def main():
    args = parse_args()
    global CACHE_MULTIPLE
    CACHE_MULTIPLE = max(1.0, args.cache_multiple)
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (multi-GPU runs are not part of it)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as ge

    pkg = ge.load_package()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if not pkg.is_built():
        ge.build()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    lib = pkg.ops()
    timer = Timer(torch, use_graph=not args.no_graph)
    loops = None
    if not args.graph:
        # K calls of the C-ABI entry point from a C++ loop between two events on
        # the launch stream (lib/libmgpu_bench_loops.so): the call rate of a
        # compiled model, which a Python caller cannot reach
        loops = pkg.bench_loops()
    bench_stream = torch.cuda.Stream()

    def ptrs(tensors):
        return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])

    K, W, R = args.steps, args.warmup, max(1, args.repeats)

    def loop_ms(call):
        """Median over R timed regions; call() runs one region of a C++ launch loop and returns its milliseconds."""
        times = [call() for _ in range(R)]
        if min(times) < 0:
            raise RuntimeError("timed launch loop failed")
        return float(np.median(times))
    only = set(filter(None, args.only.split(",")))

    def want(name):
        return not only or name in only

    def check():
        msg = lib.mgpuOpsTakeLastError()
        if msg is not None:
            raise RuntimeError(msg.decode())

    gen = torch.Generator(device=dev)
    gen.manual_seed(20241)
    kernels = []

    if args.copy_calibration:
        # A copy of known size: 64 MiB read + 64 MiB written per launch.  The
        # FETCH_SIZE / WRITE_SIZE a profiler reports for it give the factor by
        # which the same counters of the other kernels are scaled.
        src = torch.empty(64 << 20, dtype=torch.uint8, device=dev).random_(generator=gen)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    def torch_graph_us(call, ncalls):
        """Microseconds per call of `call(i)`, i = 0..ncalls-1, captured once into a graph and replayed: what the
        framework's own kernel for the same operation takes on this device (an outside reference point).  With one
        call per rotating buffer set a replay meets every set as cold as the timed loops above do.  The results of
        the captured calls are kept alive so that each call writes memory of its own.  None when torch is not asked."""
        if args.no_torch_ref:
            return None
        try:
            for i in range(min(ncalls, 3)):
                call(i)
            torch.cuda.synchronize()
            graph, side, keep = torch.cuda.CUDAGraph(), torch.cuda.Stream(), []
            with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
                for i in range(ncalls):
                    keep.append(call(i))
            graph.replay()
            torch.cuda.synchronize()
            best = None
            for _ in range(max(3, R)):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                graph.replay()
                e1.record()
                e1.synchronize()
                t = e0.elapsed_time(e1) * 1e3 / ncalls
                best = t if best is None else min(best, t)
            del graph, keep
            return best
        except Exception:
            return None

    def with_torch(entry, us_torch):
        if us_torch:
            entry["torch_us"] = round(us_torch, 3)
            entry["speedup_vs_torch"] = round(us_torch / entry.get("us_per_launch", entry["value"]), 2)
        return entry

    # ---------------- headline: LayerNorm fp32 (32,128,768) -------------------
    m, n = 32 * 128, 768
    ln_bytes = 2 * m * n * 4 + 2 * n * 4
    nsets = rotating_sets(2 * m * n * 4)
    # The rotating buffer sets of the three small configurations are consecutive pieces of one
    # allocation each, as activations out of a pooled allocator are (measured: 2 % faster than
    # one allocation per buffer, 4.98 against 5.08 us for this kernel in the same process).
    slab = torch.empty((2, nsets, m, n), device=dev)
    slab[0].normal_(generator=gen)
    xs, ys = list(slab[0]), list(slab[1])
    gamma = 1 + 0.02 * torch.randn(n, device=dev, generator=gen)
    beta = 0.02 * torch.randn(n, device=dev, generator=gen)

    def ln32(i, xs=xs, ys=ys):
        s = torch.cuda.current_stream().cuda_stream
        lib.mgpuLayerNormF32(xs[i % len(xs)].data_ptr(), gamma.data_ptr(), beta.data_ptr(),
                             ys[i % len(ys)].data_ptr(), 1e-5, m, n, s)

    if loops:
        torch.cuda.synchronize()
        sp = ctypes.c_void_p(bench_stream.cuda_stream)
        ln_args = (ctypes.c_void_p(gamma.data_ptr()), ctypes.c_void_p(beta.data_ptr()), ctypes.c_float(1e-5), m, n)
        ms_cold = loop_ms(lambda: loops.mgpuBenchLayerNormF32(ptrs(xs), ptrs(ys), nsets, *ln_args, K, W, sp))
        ms_warm = loop_ms(lambda: loops.mgpuBenchLayerNormF32(ptrs(xs[:1]), ptrs(ys[:1]), 1, *ln_args, K, W, sp))
        copy_ms = loop_ms(lambda: loops.mgpuProbeCopy(ptrs(xs), ptrs(ys), nsets, ctypes.c_size_t(m * n * 4), K, W, sp))
    else:
        ms_cold = timer.run(ln32, K, W, R)
        ms_warm = timer.run(lambda i: ln32(0), K, W, R)
    check()
    COPY_WHAT = ("plain copy kernel (one 16-byte vector per lane, non-temporal stores) over the same buffer sets: as "
                 "many bytes in and out, same rotation")
    headline = hbm_entry("layernorm_f32", "LayerNorm fp32 (32,128,768) eps=1e-5 [configs[1]]", "f32",
                         ln_bytes, ms_cold, K, ms_warm, copy_ms * 1e3 / K if loops else None, COPY_WHAT)
    with_torch(headline, torch_graph_us(lambda i: torch.nn.functional.layer_norm(xs[i], (n,), gamma, beta, 1e-5), nsets))
    del xs, ys, slab

    # The headline above is the contract's region: W untimed launches, then exactly K timed ones.  The entries
    # below keep at least the default region (200 timed launches behind 20 untimed ones; fractions of it for the
    # long kernels) whatever --steps / --warmup asked for: in a region of 20 launches of a 4 us kernel the start
    # of the queue is a tenth of the figure, and a matrix kernel has not reached the clocks it holds under
    # sustained load (fused MHA b32 s512 h12: 38.9 us at --steps 20 against 35.2 at the default).
    K_HEADLINE, W_HEADLINE = K, W
    K, W = max(K, 200), max(W, 20)

    # ---------------- LayerNorm fp16 ------------------------------------------
    if want("layernorm_f16"):
        nsets = rotating_sets(2 * m * n * 2)
        slab = torch.empty((2, nsets, m, n), device=dev, dtype=torch.float16)
        slab[0].normal_(generator=gen)
        xh, yh = list(slab[0]), list(slab[1])
        gh, bh = gamma.half(), beta.half()

        def ln16(i):
            s = torch.cuda.current_stream().cuda_stream
            lib.mgpuLayerNormF16(xh[i % nsets].data_ptr(), gh.data_ptr(), bh.data_ptr(),
                                 yh[i % nsets].data_ptr(), 1e-5, m, n, s)

        if loops:
            torch.cuda.synchronize()
            a16 = (ctypes.c_void_p(gh.data_ptr()), ctypes.c_void_p(bh.data_ptr()), ctypes.c_float(1e-5), m, n)
            ms = loop_ms(lambda: loops.mgpuBenchLayerNormF16(ptrs(xh), ptrs(yh), nsets, *a16, K, W, sp))
            msw = loop_ms(lambda: loops.mgpuBenchLayerNormF16(ptrs(xh[:1]), ptrs(yh[:1]), 1, *a16, K, W, sp))
            copy_ms = loop_ms(lambda: loops.mgpuProbeCopy(ptrs(xh), ptrs(yh), nsets, ctypes.c_size_t(m * n * 2), K, W, sp))
        else:
            ms = timer.run(ln16, K, W, R)
            msw = timer.run(lambda i: ln16(0), K, W, R)
        check()
        kernels.append(hbm_entry("layernorm_f16", "LayerNorm fp16 (32,128,768)", "f16",
                                 2 * m * n * 2 + 2 * n * 2, ms, K, msw, copy_ms * 1e3 / K if loops else None, COPY_WHAT))
        with_torch(kernels[-1], torch_graph_us(lambda i: torch.nn.functional.layer_norm(xh[i], (n,), gh, bh, 1e-5), nsets))
        del xh, yh, slab

    # ---------------- add fp32 (3,640,640) -------------------------------------
    if want("add_f32"):
        ne = 3 * 640 * 640
        nsets = rotating_sets(3 * ne * 4)
        slab = torch.empty((3, nsets, ne), device=dev)
        slab[:2].uniform_(-1.0, 1.0, generator=gen)
        aa, bb, cc = list(slab[0]), list(slab[1]), list(slab[2])

        def add(i):
            s = torch.cuda.current_stream().cuda_stream
            j = i % nsets
            lib.mgpuAddF32(aa[j].data_ptr(), bb[j].data_ptr(), cc[j].data_ptr(), ne, s)

        if loops:
            torch.cuda.synchronize()
            ms = loop_ms(lambda: loops.mgpuBenchAddF32(ptrs(aa), ptrs(bb), ptrs(cc), nsets, ctypes.c_int64(ne), K, W, sp))
            msw = loop_ms(lambda: loops.mgpuBenchAddF32(ptrs(aa[:1]), ptrs(bb[:1]), ptrs(cc[:1]), 1, ctypes.c_int64(ne), K, W, sp))
            copy_ms = loop_ms(lambda: loops.mgpuProbeCombine(ptrs(aa), ptrs(bb), ptrs(cc), nsets, ctypes.c_size_t(ne * 4),
                                                             K, W, sp))
        else:
            ms = timer.run(add, K, W, R)
            msw = timer.run(lambda i: add(0), K, W, R)
        check()
        kernels.append(hbm_entry("add_f32", "add fp32 (3,640,640) [configs[0]]", "f32", 3 * ne * 4, ms, K, msw,
                                 copy_ms * 1e3 / K if loops else None,
                                 "two-streams-in one-out probe (xor of two 16-byte vectors per lane, non-temporal store) "
                                 "over the same buffer sets"))
        with_torch(kernels[-1], torch_graph_us(lambda i: torch.add(aa[i], bb[i], out=cc[i]), nsets))
        del aa, bb, cc, slab

    # ---------------- the same two kernels where launch latency is amortised ----
    # (the configurations above move 15-25 MB per launch, a few microseconds of
    # HBM time; these move 1.6 GB and 3.2 GB)
    if want("layernorm_f32_large") and loops:
        mL = 64 * m
        xl = torch.randn((mL, n), device=dev, generator=gen)
        yl = torch.empty_like(xl)
        torch.cuda.synchronize()
        ms = loop_ms(lambda: loops.mgpuBenchLayerNormF32(ptrs([xl]), ptrs([yl]), 1, *ln_args[:3], mL, n, 20, 3, sp))
        copy_ms = loop_ms(lambda: loops.mgpuProbeCopy(ptrs([xl]), ptrs([yl]), 1, ctypes.c_size_t(mL * n * 4), 20, 3, sp))
        check()
        kernels.append(hbm_entry("layernorm_f32_large", f"LayerNorm fp32 ({mL},{n})", "f32",
                                 2 * mL * n * 4 + 2 * n * 4, ms, 20, None, copy_ms * 1e3 / 20, COPY_WHAT))
        del xl, yl
    if want("layernorm_f32_wide") and loops:
        # a wide row (an LLM hidden size): one 256-thread block holds the row in registers
        mW, nW = 4096, 8192
        nsW = rotating_sets(2 * mW * nW * 4)
        xw = [torch.randn((mW, nW), device=dev, generator=gen) for _ in range(nsW)]
        yw = [torch.empty((mW, nW), device=dev) for _ in range(nsW)]
        gw = 1 + 0.02 * torch.randn(nW, device=dev, generator=gen)
        bw = 0.02 * torch.randn(nW, device=dev, generator=gen)
        torch.cuda.synchronize()
        ms = loop_ms(lambda: loops.mgpuBenchLayerNormF32(ptrs(xw), ptrs(yw), nsW, ctypes.c_void_p(gw.data_ptr()),
                                                         ctypes.c_void_p(bw.data_ptr()), ctypes.c_float(1e-5), mW, nW, 50, 5, sp))
        copy_ms = loop_ms(lambda: loops.mgpuProbeCopy(ptrs(xw), ptrs(yw), nsW, ctypes.c_size_t(mW * nW * 4), 50, 5, sp))
        check()
        kernels.append(hbm_entry("layernorm_f32_wide", f"LayerNorm fp32 ({mW},{nW})", "f32",
                                 2 * mW * nW * 4 + 2 * nW * 4, ms, 50, None, copy_ms * 1e3 / 50, COPY_WHAT))
        del xw, yw
    if want("add_f32_large") and loops:
        nl = 1 << 28
        al, bl = torch.rand(nl, device=dev, generator=gen), torch.rand(nl, device=dev, generator=gen)
        cl = torch.empty_like(al)
        torch.cuda.synchronize()
        ms = loop_ms(lambda: loops.mgpuBenchAddF32(ptrs([al]), ptrs([bl]), ptrs([cl]), 1, ctypes.c_int64(nl), 20, 3, sp))
        copy_ms = loop_ms(lambda: loops.mgpuProbeCombine(ptrs([al]), ptrs([bl]), ptrs([cl]), 1, ctypes.c_size_t(nl * 4), 20, 3, sp))
        check()
        kernels.append(hbm_entry("add_f32_large", f"add fp32 ({nl} elements)", "f32", 3 * nl * 4, ms, 20, None,
                                 copy_ms * 1e3 / 20, "two-streams-in one-out probe over the same buffers"))
        del al, bl, cl

    # ---------------- fused MHA -------------------------------------------------
    def torch_sdpa_us(qkv, causal):
        """Microseconds per call of torch.nn.functional.scaled_dot_product_attention (flash backend) on the
        q, k, v of a packed [B, S, 3, H, D] tensor; a graph of 20 calls, the fastest of R replays.  None where this
        torch build has no such kernel for the device."""
        try:
            from torch.nn.attention import sdpa_kernel, SDPBackend
            q, k, v = [qkv[:, :, i].permute(0, 2, 1, 3).contiguous() for i in range(3)]
            with sdpa_kernel(SDPBackend.FLASH_ATTENTION):
                call = lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=causal)
                for _ in range(3):
                    call()
                torch.cuda.synchronize()
                graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
                with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
                    for _ in range(20):
                        call()
                best = None
                for _ in range(max(3, R)):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    graph.replay()
                    e1.record()
                    e1.synchronize()
                    t = e0.elapsed_time(e1) * 1e3 / 20
                    best = t if best is None else min(best, t)
            return best
        except Exception:     # no flash kernel in this build / for this device: the comparison is left out
            return None

    def fmha_case(name, workload, B, S, H, masked, D=64, causal=False):
        qkv = (torch.randn((B, S, 3, H, D), device=dev, generator=gen) / 8).half()
        out = torch.empty((B, S, H * D), device=dev, dtype=torch.float16)
        lens = None
        flop = 4.0 * B * H * S * S * D
        if masked:
            lens_cpu = torch.randint(256, 513, (B,), generator=torch.Generator().manual_seed(20244), dtype=torch.int32)
            lens = lens_cpu.to(dev)
            flop_valid = 4.0 * H * D * S * float(lens_cpu.sum())
        elif causal:
            flop_valid = 4.0 * B * H * D * (S * (S + 1) / 2)  # query i sees keys 0..i
        else:
            flop_valid = flop

        def run(i):
            s = torch.cuda.current_stream().cuda_stream
            lib.mgpuFusedMHAF16(qkv.data_ptr(), lens.data_ptr() if lens is not None else None,
                                out.data_ptr(), B, S, H, D, D ** -0.5, int(causal), s)

        steps = max(20, K // 4)
        warm = max(10, W)  # enough launches for the clocks to settle under matrix load
        if loops:
            torch.cuda.synchronize()
            ms = loop_ms(lambda: loops.mgpuBenchFusedMHAF16(
                ptrs([qkv]), ptrs([out]), 1, ctypes.c_void_p(lens.data_ptr() if lens is not None else None),
                B, S, H, D, ctypes.c_float(D ** -0.5), int(causal), steps, warm, sp))
        else:
            ms = timer.run(run, steps, warm, R)
        check()
        us = ms * 1e3 / steps
        tf = flop_valid / us / 1e6
        nbytes = qkv.numel() * 2 + out.numel() * 2 + (4 * B if masked else 0)
        entry = {"name": name, "workload": workload, "dtype": "f16", "metric": "TFLOP/s", "value": round(tf, 1),
                 "us_per_launch": round(us, 3),
                 "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                              "unit": "TFLOP/s", "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4),
                              "traffic": TRAFFIC_BYTES.get(name)},
                 "algorithmic_flop": flop_valid, "algorithmic_bytes": nbytes,
                 "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        if masked or causal:
            entry["dense_flop"] = flop
        if not masked and not args.no_sdpa:
            # what the framework's own attention (torch SDPA, flash backend) takes on this device for the same
            # problem, from contiguous [B, H, S, D] operands: an outside reference point, not a ceiling
            ref_us = torch_sdpa_us(qkv, causal)
            entry["torch_sdpa_us"] = ref_us and round(ref_us, 2)
            entry["speedup_vs_torch_sdpa"] = ref_us and round(ref_us / us, 2)
        kernels.append(entry)

    if want("fmha_b32_s128"):
        fmha_case("fmha_b32_s128", "fused MHA fp16 b32 s128 h12 d64 [configs[2]]", 32, 128, 12, False)
    if want("fmha_b8_s512_masked"):
        fmha_case("fmha_b8_s512_masked", "fused MHA fp16 b8 s512 h16 d64, key lengths U[256,512] [configs[3]]",
                  8, 512, 16, True)
    if want("fmha_b32_s512"):
        fmha_case("fmha_b32_s512", "fused MHA fp16 b32 s512 h12 d64 [roofline target shape]", 32, 512, 12, False)

    if want("fmha_b32_s512_causal"):
        fmha_case("fmha_b32_s512_causal", "fused MHA fp16 b32 s512 h12 d64, causal (the reference layer's mask)",
                  32, 512, 12, False, causal=True)

    if want("fmha_d128_b32_s512"):
        fmha_case("fmha_d128_b32_s512", "fused MHA fp16 b32 s512 h8 d128 [the reference layer's head geometry]",
                  32, 512, 8, False, D=128)

    if want("fmha_d128_b4_s2048"):
        fmha_case("fmha_d128_b4_s2048", "fused MHA fp16 b4 s2048 h32 d128 [long sequences, the reference layer's head size]",
                  4, 2048, 32, False, D=128)

    if want("fmha_b4_s4096"):
        fmha_case("fmha_b4_s4096", "fused MHA fp16 b4 s4096 h16 d64 [long sequences: 64 queries per wavefront]",
                  4, 4096, 16, False)
    if want("fmha_d256_b4_s2048"):
        fmha_case("fmha_d256_b4_s2048", "fused MHA fp16 b4 s2048 h8 d256 [the widest head of the reference's kernel list]",
                  4, 2048, 8, False, D=256)

    # ---------------- GEMM with fused epilogue ---------------------------------
    # The four GEMMs of the BERT-base layer at 4096 tokens.  mgpuMatmulExF16 runs whichever of the library (+ a
    # separate GELU pass where there is one) and the hand-written MFMA kernel the committed table names for the
    # shape; mgpuGemmMfmaF16 is the hand-written kernel by itself.  With --tune-gemm the shape is first measured
    # on this device (mgpuBenchTuneMatmulEx of the launch-loop library) and the table line that measurement gives is printed.
    def tune_shape(M_, N_, K_, has_bias, act, residual):
        """Measure one shape on this device and print the line of gemm_table.inc that the measurement gives."""
        times = (ctypes.c_float * 4)()
        index, version = ctypes.c_int32(-1), ctypes.c_int32(0)
        kept = int(pkg.bench_loops().mgpuBenchTuneMatmulEx(1, M_, N_, K_, has_bias, act, residual, times,
                                                           ctypes.byref(index), ctypes.byref(version)))
        if kept < 0:
            raise RuntimeError("mgpuBenchTuneMatmulEx failed")
        print(f"{{1, {M_}, {N_}, {K_}, {has_bias}, {act}, {residual}, {kept & 1}, {kept >> 1}}},  // library "
              f"{times[0]:.1f} us (the best of its 64 answers {times[3]:.1f}: solution {index.value} of hipBLASLt "
              f"{version.value}), hand-written {times[1]:.1f} us, library on a K-major weight {times[2]:.1f} us",
              file=sys.stderr)
        kept &= 1
        return kept

    if args.tune_gemm and want("decoding_layer"):
        # the four GEMMs of the decoding layer below (4096 tokens, d_model 2048, feed-forward 2048)
        tune_shape(4096, 6144, 2048, 0, 0, 0)
        tune_shape(4096, 2048, 2048, 1, 0, 0)
        tune_shape(4096, 2048, 2048, 1, 1, 0)
        tune_shape(4096, 2048, 2048, 1, 0, 1)

    def gemm_case(name, workload, M_, K_, N_, act, residual):
        x = torch.randn((M_, K_), device=dev, generator=gen).half()
        wt = (0.02 * torch.randn((K_, N_), device=dev, generator=gen)).half()
        bias = (0.02 * torch.randn((N_,), device=dev, generator=gen)).half()
        res = torch.randn((M_, N_), device=dev, generator=gen).half() if residual else None
        y = torch.empty((M_, N_), device=dev, dtype=torch.float16)

        def gemm(fn):
            def run(i):
                fn(x.data_ptr(), wt.data_ptr(), bias.data_ptr(), y.data_ptr(), res.data_ptr() if residual else None,
                   M_, N_, K_, 1, act, int(residual), torch.cuda.current_stream().cuda_stream)
            run(0)                       # first use of the shape (descriptors, code), untimed
            torch.cuda.synchronize()
            steps = max(20, K // 4)
            ms = Timer(torch, use_graph=True).run(run, steps, 3, R)
            check()
            return ms * 1e3 / steps

        tuned = tune_shape(M_, N_, K_, 1, act, int(residual)) if args.tune_gemm else None
        us_auto, us_mfma = gemm(lib.mgpuMatmulExF16), gemm(lib.mgpuGemmMfmaF16)
        wt = pkg.pack_weight(wt)        # the K-major copy a caller with constant weights makes once
        us_packed = gemm(lib.mgpuMatmulExPackedF16)
        flop = 2.0 * M_ * N_ * K_
        kernels.append({"name": name, "workload": workload,
                        "dtype": "f16", "metric": "TFLOP/s", "value": round(flop / us_auto / 1e6, 1),
                        "us_per_launch": round(us_auto, 2), "us_per_launch_gemm_mfma": round(us_mfma, 2),
                        "us_per_launch_packed_weight": round(us_packed, 2),
                        "kernel_kept_by_tuning_in_this_run": tuned if tuned is None else ("gemm_mfma" if tuned else "library"),
                        "roofline": {"bound": "mfma", "achieved": round(flop / us_auto / 1e6, 1),
                                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(flop / us_auto / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None},
                        "algorithmic_flop": flop})

    if want("gemm_qkv"):
        gemm_case("gemm_qkv", "GEMM fp16 4096x768 . 768x2304 + bias (QKV of configs[4])", 4096, 768, 2304, 0, False)
    if want("gemm_proj"):
        gemm_case("gemm_proj", "GEMM fp16 4096x768 . 768x768 + bias (projection of configs[4])", 4096, 768, 768, 0, False)
    if want("gemm_ffn1_gelu"):
        gemm_case("gemm_ffn1_gelu", "GEMM fp16 4096x768 . 768x3072 + bias + erf-GELU (FFN1 of configs[4])",
                  4096, 768, 3072, 2, False)
    if want("gemm_ffn2"):
        gemm_case("gemm_ffn2", "GEMM fp16 4096x3072 . 3072x768 + bias (FFN2 of configs[4])", 4096, 3072, 768, 0, False)

    # ---------------- BERT-base encoder layer ----------------------------------
    if want("bert_layer"):
        B, S, d, ffn, H = 32, 128, 768, 3072, 12

        def w(*shape, s=0.02):
            return (s * torch.randn(shape, device=dev, generator=gen)).half()

        x = torch.randn((B, S, d), device=dev, generator=gen).half()
        P = [w(d, 3 * d), w(3 * d), w(d, d), w(d), (1 + w(d).float()).half(), w(d), w(d, ffn), w(ffn),
             w(ffn, d), w(d), (1 + w(d).float()).half(), w(d)]
        out = torch.empty_like(x)

        def layer(i):
            s = torch.cuda.current_stream().cuda_stream
            lib.mgpuBertEncoderLayerF16(x.data_ptr(), *[p.data_ptr() for p in P], None, out.data_ptr(),
                                        B, S, d, ffn, H, 1e-5, s)

        steps = max(10, K // 10)
        us_no_alloc = us_cached = None
        if loops:
            # the calls come from a C++ loop, like a compiled model's: seven kernels per call
            layer(0)  # first use of the GEMM shapes, untimed
            torch.cuda.synchronize()
            largs = (ctypes.c_void_p(x.data_ptr()), ptrs(P), None, ctypes.c_void_p(out.data_ptr()),
                     ctypes.c_int64(B), ctypes.c_int64(S), ctypes.c_int64(d), ctypes.c_int64(ffn), ctypes.c_int64(H),
                     ctypes.c_float(1e-5))
            # A timed region of this entry is only 23 calls (2.6 ms) and seven of them end before the
            # device has settled into the clocks it holds under sustained matrix work (the first
            # regions measure 3-6 % longer than those 30 ms later): 200 untimed calls come first.
            loops.mgpuBenchBertEncoderLayerF16(*largs, 0, 200, 0, sp)
            ms = loop_ms(lambda: loops.mgpuBenchBertEncoderLayerF16(*largs, 0, steps, 3, sp))
            us_no_alloc = loop_ms(lambda: loops.mgpuBenchBertEncoderLayerF16(*largs, 1, steps, 3, sp)) * 1e3 / steps
            # with the weight cache on, the GEMMs that the library runs fastest on a K-major weight get the
            # cache's transposed copy
            lib.mgpuLLMOpsCacheWeights(1)
            try:
                layer(0)
                torch.cuda.synchronize()
                loops.mgpuBenchBertEncoderLayerF16(*largs, 0, 200, 0, sp)   # (sustained clocks, as above)
                us_cached = loop_ms(lambda: loops.mgpuBenchBertEncoderLayerF16(*largs, 0, steps, 3, sp)) * 1e3 / steps
            finally:
                lib.mgpuLLMOpsCacheWeights(0)
        else:
            ms = Timer(torch, use_graph=False).run(layer, steps, 3, R)
        check()
        us = ms * 1e3 / steps
        flop = 2.0 * B * S * d * (3 * d + d + ffn + ffn) + 4.0 * B * H * S * S * 64
        def torch_bert(i):
            F_ = torch.nn.functional
            wqkv, bqkv, wo, bo, g1, be1, w1, b1, w2, b2, g2, be2 = P
            qkv_ = torch.addmm(bqkv, x.view(-1, d), wqkv).view(B, S, 3, H, d // H)
            q_, k_, v_ = [qkv_[:, :, j].transpose(1, 2) for j in range(3)]
            ctx = F_.scaled_dot_product_attention(q_, k_, v_).transpose(1, 2).reshape(-1, d)
            h1 = F_.layer_norm(torch.addmm(bo, ctx, wo) + x.view(-1, d), (d,), g1, be1, 1e-5)
            f_ = F_.gelu(torch.addmm(b1, h1, w1))
            return F_.layer_norm(torch.addmm(b2, f_, w2) + h1, (d,), g2, be2, 1e-5)

        us_torch = torch_graph_us(torch_bert, 10)
        kernels.append({"name": "bert_layer", "workload": "BERT-base encoder layer fp16 (32,128,768) [configs[4]]",
                        "dtype": "f16", "metric": "us", "value": round(us, 1), "higher_is_better": False,
                        "us_per_call_no_alloc_entry_point": us_no_alloc and round(us_no_alloc, 1),
                        "us_per_call_with_weight_cache": us_cached and round(us_cached, 1),
                        "torch_us": us_torch and round(us_torch, 1),
                        "speedup_vs_torch": us_torch and round(us_torch / us, 2),
                        "roofline": {"bound": "mfma", "achieved": round(flop / us / 1e6, 1),
                                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(flop / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None},
                        "algorithmic_flop": flop})

    if want("decoding_layer"):
        # mgpuLLMDecodingContextLayer at the geometry of the reference's own benchmark layer
        # (benchmark/PyTorch/Models/LLM.py: d_model 2048, 16 heads of 128, feed-forward 2048, causal, ReLU)
        B, S, d, ffn, H = 8, 512, 2048, 2048, 16

        def f(*shape, s=0.02):
            return s * torch.randn(shape, device=dev, generator=gen)

        x = torch.randn((B, S, d), device=dev, generator=gen)
        P = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
        out = torch.empty_like(x)

        def dec(i):
            lib.mgpuLLMDecodingContextLayer(x.data_ptr(), *[p.data_ptr() for p in P], out.data_ptr(), B, S, d, ffn, H,
                                            True, True, True, torch.cuda.current_stream().cuda_stream)

        steps = max(10, K // 10)
        ms = Timer(torch, use_graph=False).run(dec, steps, 3, R)
        check()
        lib.mgpuLLMOpsCacheWeights(1)   # the weights cast to fp16 once instead of on every call
        try:
            dec(0)
            us_cached = Timer(torch, use_graph=False).run(dec, steps, 3, R) * 1e3 / steps
        finally:
            lib.mgpuLLMOpsCacheWeights(0)
        check()
        us = ms * 1e3 / steps
        flop = 2.0 * B * S * d * (3 * d + d + 2 * ffn) + 4.0 * B * H * (d // H) * (S * (S + 1) / 2)

        # the same pre-LN layer composed from torch's own operators, weights cast to fp16 beforehand (the layer the
        # reference's PyTorch benchmark builds: benchmark/PyTorch/Models/LLM.py, TransformerEncoderLayer(2048, 16,
        # norm_first) under a causal mask)
        Ph = [p.half() for p in P]

        def torch_dec(i):
            F_ = torch.nn.functional
            wqkv, wo, bo, w1, b1, w2, b2 = Ph
            x16 = x.view(-1, d).half()
            qkv_ = (F_.layer_norm(x16, (d,)) @ wqkv).view(B, S, 3, H, d // H)
            q_, k_, v_ = [qkv_[:, :, j].transpose(1, 2) for j in range(3)]
            ctx = F_.scaled_dot_product_attention(q_, k_, v_, is_causal=True).transpose(1, 2).reshape(-1, d)
            y = x16 + torch.addmm(bo, ctx, wo)
            f_ = torch.relu(torch.addmm(b1, F_.layer_norm(y, (d,)), w1))
            return (y + torch.addmm(b2, f_, w2)).float()

        us_torch = torch_graph_us(torch_dec, 10)
        kernels.append({"name": "decoding_layer",
                        "workload": "mgpuLLMDecodingContextLayer fp32 in/out (8,512,2048), 16 heads of 128, ffn 2048, "
                                    "causal, ReLU; fp32 weights cast to fp16 on every call, as in the reference",
                        "dtype": "f16", "metric": "us", "value": round(us, 1), "higher_is_better": False,
                        "us_per_call_with_weight_cache": round(us_cached, 1),
                        "torch_us": us_torch and round(us_torch, 1),
                        "speedup_vs_torch": us_torch and round(us_torch / us, 2),
                        "speedup_vs_torch_with_weight_cache": us_torch and round(us_torch / us_cached, 2),
                        "roofline": {"bound": "mfma", "achieved": round(flop / us / 1e6, 1),
                                     "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": round(flop / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None},
                        "algorithmic_flop": flop})

    if want("conv2d"):
        # the shape of the reference's End2End conv test: 16x3x256x256 -> 64 channels, 3x3, pad 1
        N_, IC, H_, W_, OC = 16, 3, 256, 256, 64
        xc = torch.randn((N_, IC, H_, W_), device=dev, generator=gen)
        wc = 0.1 * torch.randn((OC, IC, 3, 3), device=dev, generator=gen)
        bc = torch.randn(OC, device=dev, generator=gen)
        yc = torch.empty((N_, OC, H_, W_), device=dev)

        def conv(i):
            lib.mgpuConv2d(xc.data_ptr(), wc.data_ptr(), bc.data_ptr(), yc.data_ptr(), None, N_, IC, H_, W_, OC, 3, 3,
                           H_, W_, 1, 1, 1, 1, 1, 1, 1, 1, False, False, torch.cuda.current_stream().cuda_stream)

        steps = max(10, K // 10)
        ms = Timer(torch, use_graph=False).run(conv, steps, 3, R)
        check()
        us = ms * 1e3 / steps
        nbytes = (xc.numel() + wc.numel() + bc.numel() + yc.numel()) * 4
        flop = 2.0 * N_ * OC * H_ * W_ * IC * 9
        kernels.append({"name": "conv2d", "workload": "conv2d fp32 16x3x256x256 -> 64, 3x3 pad 1", "dtype": "f32",
                        "metric": "us", "value": round(us, 1), "higher_is_better": False,
                        "roofline": {"bound": "hbm", "achieved": round(nbytes / us / 1e3, 1), "peak": HBM_PEAK_GBS,
                                     "unit": "GB/s", "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "traffic": None},
                        "algorithmic_bytes": nbytes, "algorithmic_flop": flop})

    # ---------------- ceilings measured in this run ------------------------------
    ceilings = None
    if loops and not args.no_ceilings:
        ceilings = measure_ceilings(torch, loops, dev, gen, sp, ptrs, R)

    phases = fmha_phases(torch, lib, pkg.bench_loops(), dev, gen) if args.fmha_phases else None

    # ---------------- CPU baseline: the CPU op library on the host cores --------
    cpu = None
    if not args.no_cpu:
        cpu_all = cpu_baselines(pkg, m, n, ln_bytes)
        cpu = cpu_all.pop("layernorm_f32")
        for e in kernels:
            key = {"add_f32": "add_f32", "fmha_b32_s128": "fmha_b32_s128", "bert_layer": "bert_layer"}.get(e["name"])
            if key and key in cpu_all:
                e["cpu_baseline"] = cpu_all[key]

    runner = None if args.no_runner else runner_end_to_end(pkg)

    # The figures the north star names, gathered once more as the LAST keys of the line so that a
    # reader who keeps only the tail of it still has them.
    def star(e, flops=False):
        if e is None:
            return None
        r = {"us_per_launch": e["us_per_launch"], e["metric"]: e["value"], "frac_of_peak": e["roofline"]["frac"]}
        if "frac_of_copy_ceiling" in e:
            r["copy_ceiling_GBs"] = e["copy_ceiling_GBs"]
            r["frac_of_copy_ceiling"] = e["frac_of_copy_ceiling"]
        if "cache_resident" in e:
            r["cache_resident_us_per_launch"] = e["cache_resident"]["us_per_launch"]
        if "hbm_frac" in e:
            r["hbm_frac"] = e["hbm_frac"]
        for key in ("torch_sdpa_us", "torch_us"):
            if e.get(key):
                r[key] = e[key]
        return r
    by_name = {e["name"]: e for e in kernels}
    north_star = {"layernorm_f32": star(headline), "layernorm_f16": star(by_name.get("layernorm_f16")),
                  "add_f32": star(by_name.get("add_f32")), "fmha_b32_s512": star(by_name.get("fmha_b32_s512")),
                  "fmha_b32_s128": star(by_name.get("fmha_b32_s128")),
                  "fmha_b8_s512_masked": star(by_name.get("fmha_b8_s512_masked")),
                  "bert_layer_us": by_name["bert_layer"]["value"] if "bert_layer" in by_name else None,
                  "bert_layer_us_with_weight_cache": by_name.get("bert_layer", {}).get("us_per_call_with_weight_cache"),
                  "bert_layer_torch_us": by_name.get("bert_layer", {}).get("torch_us"),
                  "decoding_layer_us": by_name["decoding_layer"]["value"] if "decoding_layer" in by_name else None,
                  "decoding_layer_us_with_weight_cache": by_name.get("decoding_layer", {}).get("us_per_call_with_weight_cache"),
                  "decoding_layer_torch_us": by_name.get("decoding_layer", {}).get("torch_us"),
                  "peaks": {"hbm_GBs": HBM_PEAK_GBS, "mfma_f16_TFLOPs": MFMA_F16_PEAK_TFLOPS}}

    result = {
        "metric": "LayerNorm GB/s (fp32 (32,128,768)); fMHA TFLOP/s and BERT-base layer us under 'kernels'",
        "value": headline["value"], "unit": "GB/s", "n_gpus": 1, "steps": K_HEADLINE, "warmup": W_HEADLINE,
        "ms_per_step": round(ms_cold / K_HEADLINE, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": headline["workload"], "rows": m, "cols": n, "eps": 1e-5,
                   "launch_mode": ("C++ loop of K calls of the C-ABI entry point" if loops else
                                   "direct ctypes launches" if args.no_graph else "hipGraph of K ctypes launches"),
                   "buffer_sets": rotating_sets(2 * m * n * 4)},
        "repeats": R, "steps_of_the_other_entries": K, "warmup_of_the_other_entries": W,
        "roofline": headline["roofline"], "cache_resident": headline.get("cache_resident"),
        "copy_ceiling": headline.get("copy_ceiling"), "frac_of_copy_ceiling": headline.get("frac_of_copy_ceiling"),
        "torch_us": headline.get("torch_us"), "speedup_vs_torch": headline.get("speedup_vs_torch"),
        "traffic_counted_at_commit": TRAFFIC_COMMIT,
        "cpu_baseline": cpu, "ceilings": ceilings, "fmha_phases": phases, "kernels": kernels,
        "runner_end_to_end": runner,
        "device": torch.cuda.get_device_name(0),
        "device_info": device_info(torch),
        "north_star": north_star,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
