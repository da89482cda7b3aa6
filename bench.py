#!/usr/bin/env python3
"""Benchmark of the device kernel library on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input, with
all inputs already resident in HBM when the timed region starts.  The headline
workload is the LayerNorm configuration of BASELINE.json (configs[1]:
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

The CPU baseline times the oracle (a plain C port of the reference semantics)
on the host cores for a bounded sample; it is a reported baseline, not the
target.
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
# HBM bytes per launch, from two rocprofv3 --pmc passes over this script
# (FETCH_SIZE scaled by 2.0, WRITE_SIZE by 1.0, the factors a 64 MiB device copy
# gives for the same counters); see profiles/layernorm_f32_hbm_traffic.md for the
# headline kernel and profiles/bench_all_configs_hbm_traffic.md for the others.
LN_F32_TRAFFIC_BYTES = 25_250_000
TRAFFIC_BYTES = {
    "layernorm_f16": 12_655_000,
    "add_f32": 14_762_000,
    "layernorm_f32_large": 1_610_400_000,
    "add_f32_large": 3_220_200_000,
    "fmha_b32_s128": 25_310_000,
    "fmha_b8_s512_masked": 31_870_000,
    "fmha_b32_s512": 100_780_000,
    "fmha_d128_b32_s512": 134_300_000,
}
# (fmha_b32_s512_causal, fmha_d128_b4_s2048, conv2d and the layers have no counter run behind them: traffic null)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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

    def run(self, fn, steps: int, warmup: int) -> float:
        """Returns elapsed milliseconds for exactly `steps` launches."""
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
    """Number of buffer sets whose total footprint exceeds the Infinity Cache."""
    return max(2, (MALL_BYTES + bytes_per_set - 1) // bytes_per_set + 2)


def hbm_entry(name, workload, dtype, bytes_per_launch, ms, steps, warm_ms=None):
    us = ms * 1e3 / steps
    gbs = bytes_per_launch / us / 1e3
    e = {"name": name, "workload": workload, "dtype": dtype, "metric": "GB/s", "value": round(gbs, 1),
         "us_per_launch": round(us, 3),
         "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                      "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_BYTES.get(name)},
         "algorithmic_bytes": bytes_per_launch}
    if warm_ms is not None:
        wus = warm_ms * 1e3 / steps
        e["cache_resident"] = {"us_per_launch": round(wus, 3), "GB/s": round(bytes_per_launch / wus / 1e3, 1)}
    return e


def main():
    args = parse_args()
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
        loops = ctypes.CDLL(os.path.join(pkg.LIB_DIR, "libmgpu_bench_loops.so"))
        for fn in ("mgpuBenchLayerNormF32", "mgpuBenchLayerNormF16", "mgpuBenchAddF32", "mgpuBenchFusedMHAF16"):
            getattr(loops, fn).restype = ctypes.c_float
    bench_stream = torch.cuda.Stream()

    def ptrs(tensors):
        return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])

    def loop_ms(ms):
        if ms < 0:
            raise RuntimeError("timed launch loop failed")
        return ms
    K, W = args.steps, args.warmup
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

    # ---------------- headline: LayerNorm fp32 (32,128,768) -------------------
    m, n = 32 * 128, 768
    ln_bytes = 2 * m * n * 4 + 2 * n * 4
    nsets = rotating_sets(2 * m * n * 4)
    xs = [torch.randn((m, n), device=dev, generator=gen) for _ in range(nsets)]
    ys = [torch.empty((m, n), device=dev) for _ in range(nsets)]
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
        ms_cold = loop_ms(loops.mgpuBenchLayerNormF32(ptrs(xs), ptrs(ys), nsets, *ln_args, K, W, sp))
        ms_warm = loop_ms(loops.mgpuBenchLayerNormF32(ptrs(xs[:1]), ptrs(ys[:1]), 1, *ln_args, K, W, sp))
    else:
        ms_cold = timer.run(ln32, K, W)
        ms_warm = timer.run(lambda i: ln32(0), K, W)
    check()
    headline = hbm_entry("layernorm_f32", "LayerNorm fp32 (32,128,768) eps=1e-5 [configs[1]]", "f32",
                         ln_bytes, ms_cold, K, ms_warm)
    headline["roofline"]["traffic"] = LN_F32_TRAFFIC_BYTES
    del xs, ys

    # ---------------- LayerNorm fp16 ------------------------------------------
    if want("layernorm_f16"):
        nsets = rotating_sets(2 * m * n * 2)
        xh = [torch.randn((m, n), device=dev, generator=gen).half() for _ in range(nsets)]
        yh = [torch.empty((m, n), device=dev, dtype=torch.float16) for _ in range(nsets)]
        gh, bh = gamma.half(), beta.half()

        def ln16(i):
            s = torch.cuda.current_stream().cuda_stream
            lib.mgpuLayerNormF16(xh[i % nsets].data_ptr(), gh.data_ptr(), bh.data_ptr(),
                                 yh[i % nsets].data_ptr(), 1e-5, m, n, s)

        if loops:
            torch.cuda.synchronize()
            a16 = (ctypes.c_void_p(gh.data_ptr()), ctypes.c_void_p(bh.data_ptr()), ctypes.c_float(1e-5), m, n)
            ms = loop_ms(loops.mgpuBenchLayerNormF16(ptrs(xh), ptrs(yh), nsets, *a16, K, W, sp))
            msw = loop_ms(loops.mgpuBenchLayerNormF16(ptrs(xh[:1]), ptrs(yh[:1]), 1, *a16, K, W, sp))
        else:
            ms = timer.run(ln16, K, W)
            msw = timer.run(lambda i: ln16(0), K, W)
        check()
        kernels.append(hbm_entry("layernorm_f16", "LayerNorm fp16 (32,128,768)", "f16",
                                 2 * m * n * 2 + 2 * n * 2, ms, K, msw))
        del xh, yh

    # ---------------- add fp32 (3,640,640) -------------------------------------
    if want("add_f32"):
        ne = 3 * 640 * 640
        nsets = rotating_sets(3 * ne * 4)
        aa = [torch.rand(ne, device=dev, generator=gen) * 2 - 1 for _ in range(nsets)]
        bb = [torch.rand(ne, device=dev, generator=gen) * 2 - 1 for _ in range(nsets)]
        cc = [torch.empty(ne, device=dev) for _ in range(nsets)]

        def add(i):
            s = torch.cuda.current_stream().cuda_stream
            j = i % nsets
            lib.mgpuAddF32(aa[j].data_ptr(), bb[j].data_ptr(), cc[j].data_ptr(), ne, s)

        if loops:
            torch.cuda.synchronize()
            ms = loop_ms(loops.mgpuBenchAddF32(ptrs(aa), ptrs(bb), ptrs(cc), nsets, ctypes.c_int64(ne), K, W, sp))
            msw = loop_ms(loops.mgpuBenchAddF32(ptrs(aa[:1]), ptrs(bb[:1]), ptrs(cc[:1]), 1, ctypes.c_int64(ne), K, W, sp))
        else:
            ms = timer.run(add, K, W)
            msw = timer.run(lambda i: add(0), K, W)
        check()
        kernels.append(hbm_entry("add_f32", "add fp32 (3,640,640) [configs[0]]", "f32", 3 * ne * 4, ms, K, msw))
        del aa, bb, cc

    # ---------------- the same two kernels where launch latency is amortised ----
    # (the configurations above move 15-25 MB per launch, a few microseconds of
    # HBM time; these move 1.6 GB and 3.2 GB)
    if want("layernorm_f32_large") and loops:
        mL = 64 * m
        xl = torch.randn((mL, n), device=dev, generator=gen)
        yl = torch.empty_like(xl)
        torch.cuda.synchronize()
        ms = loop_ms(loops.mgpuBenchLayerNormF32(ptrs([xl]), ptrs([yl]), 1, *ln_args[:3], mL, n, 20, 3, sp))
        check()
        kernels.append(hbm_entry("layernorm_f32_large", f"LayerNorm fp32 ({mL},{n})", "f32",
                                 2 * mL * n * 4 + 2 * n * 4, ms, 20))
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
        ms = loop_ms(loops.mgpuBenchLayerNormF32(ptrs(xw), ptrs(yw), nsW, ctypes.c_void_p(gw.data_ptr()),
                                                 ctypes.c_void_p(bw.data_ptr()), ctypes.c_float(1e-5), mW, nW, 50, 5, sp))
        check()
        kernels.append(hbm_entry("layernorm_f32_wide", f"LayerNorm fp32 ({mW},{nW})", "f32",
                                 2 * mW * nW * 4 + 2 * nW * 4, ms, 50))
        del xw, yw
    if want("add_f32_large") and loops:
        nl = 1 << 28
        al, bl = torch.rand(nl, device=dev, generator=gen), torch.rand(nl, device=dev, generator=gen)
        cl = torch.empty_like(al)
        torch.cuda.synchronize()
        ms = loop_ms(loops.mgpuBenchAddF32(ptrs([al]), ptrs([bl]), ptrs([cl]), 1, ctypes.c_int64(nl), 20, 3, sp))
        check()
        kernels.append(hbm_entry("add_f32_large", f"add fp32 ({nl} elements)", "f32", 3 * nl * 4, ms, 20))
        del al, bl, cl

    # ---------------- fused MHA -------------------------------------------------
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
        if loops:
            torch.cuda.synchronize()
            ms = loop_ms(loops.mgpuBenchFusedMHAF16(
                ptrs([qkv]), ptrs([out]), 1, ctypes.c_void_p(lens.data_ptr() if lens is not None else None),
                B, S, H, D, ctypes.c_float(D ** -0.5), int(causal), steps, max(3, W // 4), sp))
        else:
            ms = timer.run(run, steps, max(3, W // 4))
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

    # ---------------- GEMM with fused epilogue ---------------------------------
    # The four GEMMs of the BERT-base layer at 4096 tokens.  mgpuMatmulExF16 runs whichever of the library (+ a
    # separate GELU pass where there is one) and the hand-written MFMA kernel its first-use measurement kept;
    # mgpuGemmMfmaF16 is the hand-written kernel by itself.
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
            run(0)                       # first use of the shape: the selection runs here, untimed
            torch.cuda.synchronize()
            steps = max(20, K // 4)
            ms = Timer(torch, use_graph=True).run(run, steps, 3)
            check()
            return ms * 1e3 / steps

        us_auto, us_mfma = gemm(lib.mgpuMatmulExF16), gemm(lib.mgpuGemmMfmaF16)
        flop = 2.0 * M_ * N_ * K_
        kernels.append({"name": name, "workload": workload,
                        "dtype": "f16", "metric": "TFLOP/s", "value": round(flop / us_auto / 1e6, 1),
                        "us_per_launch": round(us_auto, 2), "us_per_launch_gemm_mfma": round(us_mfma, 2),
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
        ms = Timer(torch, use_graph=False).run(layer, steps, 3)
        check()
        us = ms * 1e3 / steps
        flop = 2.0 * B * S * d * (3 * d + d + ffn + ffn) + 4.0 * B * H * S * S * 64
        kernels.append({"name": "bert_layer", "workload": "BERT-base encoder layer fp16 (32,128,768) [configs[4]]",
                        "dtype": "f16", "metric": "us", "value": round(us, 1), "higher_is_better": False,
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
        ms = Timer(torch, use_graph=False).run(dec, steps, 3)
        check()
        us = ms * 1e3 / steps
        flop = 2.0 * B * S * d * (3 * d + d + 2 * ffn) + 4.0 * B * H * (d // H) * (S * (S + 1) / 2)
        kernels.append({"name": "decoding_layer",
                        "workload": "mgpuLLMDecodingContextLayer fp32 in/out (8,512,2048), 16 heads of 128, ffn 2048, "
                                    "causal, ReLU; fp32 weights cast to fp16 on every call, as in the reference",
                        "dtype": "f16", "metric": "us", "value": round(us, 1), "higher_is_better": False,
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
        ms = Timer(torch, use_graph=False).run(conv, steps, 3)
        check()
        us = ms * 1e3 / steps
        nbytes = (xc.numel() + wc.numel() + bc.numel() + yc.numel()) * 4
        flop = 2.0 * N_ * OC * H_ * W_ * IC * 9
        kernels.append({"name": "conv2d", "workload": "conv2d fp32 16x3x256x256 -> 64, 3x3 pad 1", "dtype": "f32",
                        "metric": "us", "value": round(us, 1), "higher_is_better": False,
                        "roofline": {"bound": "hbm", "achieved": round(nbytes / us / 1e3, 1), "peak": HBM_PEAK_GBS,
                                     "unit": "GB/s", "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "traffic": None},
                        "algorithmic_bytes": nbytes, "algorithmic_flop": flop})

    # ---------------- CPU baseline: the oracle on the host cores ---------------
    cpu = None
    if not args.no_cpu:
        oracle = ge.load_oracle()
        rng = np.random.default_rng(20241)
        x = rng.standard_normal((m, n)).astype(np.float32)
        g = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
        b = (0.02 * rng.standard_normal(n)).astype(np.float32)
        threads = oracle.num_threads()
        oracle.layernorm(x, g, b)
        reps, t0 = 0, time.perf_counter()
        while reps < 2000 and time.perf_counter() - t0 < 10.0:
            oracle.layernorm(x, g, b)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        cpu = {"value": round(ln_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": f"{reps} passes of LayerNorm fp32 (32,128,768) through oracle_layernorm "
                         f"(fp64 arithmetic, OpenMP, {threads} threads), {dt * 1e6:.0f} us per pass"}

    result = {
        "metric": "LayerNorm GB/s (fp32 (32,128,768)); fMHA TFLOP/s and BERT-base layer us under 'kernels'",
        "value": headline["value"], "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_cold / K, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": headline["workload"], "rows": m, "cols": n, "eps": 1e-5,
                   "launch_mode": ("C++ loop of K calls of the C-ABI entry point" if loops else
                                   "direct ctypes launches" if args.no_graph else "hipGraph of K ctypes launches"),
                   "buffer_sets": rotating_sets(2 * m * n * 4)},
        "roofline": headline["roofline"], "cache_resident": headline.get("cache_resident"),
        "cpu_baseline": cpu, "kernels": kernels,
        "device": torch.cuda.get_device_name(0),
        "device_info": device_info(torch),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
