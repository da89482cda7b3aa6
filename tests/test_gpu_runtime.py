"""The mgpu* device runtime C ABI on a real GPU, and the GPU runner end to end."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(ROOT, "multi-device-model-compiler_amd", "tools"))
import gen_data  # noqa: E402


@pytest.fixture(scope="module")
def rt(pkg, gpu):
    return pkg.runtime()


def host_ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def test_alloc_copy_memset_roundtrip(rt):
    s = rt.mgpuStreamCreate()
    n = 1 << 16
    a = np.arange(n, dtype=np.float32)
    out = np.zeros(n, np.float32)
    d = rt.mgpuMemAlloc(n * 4, s)
    assert d
    rt.mgpuMemcpy(d, host_ptr(a), n * 4, s)
    rt.mgpuMemcpy(host_ptr(out), d, n * 4, s)
    rt.mgpuStreamSynchronize(s)
    assert np.array_equal(a, out)
    rt.mgpuMemset32(d, 0x3F800000, n, s)  # 1.0f
    rt.mgpuMemcpy(host_ptr(out), d, n * 4, s)
    rt.mgpuStreamSynchronize(s)
    assert np.all(out == 1.0)
    h = np.zeros(n, np.uint16)
    rt.mgpuMemset16(d, 0x3C00, n, s)
    rt.mgpuMemcpy(host_ptr(h), d, n * 2, s)
    rt.mgpuStreamSynchronize(s)
    assert np.all(h == 0x3C00)
    rt.mgpuMemFree(d, s)
    d2 = rt.mgpuMemAllocAsync(4096, s)
    rt.mgpuMemFreeAsync(d2, s)
    rt.mgpuStreamSynchronize(s)
    rt.mgpuStreamDestroy(s)
    assert rt.mgpuRuntimeTakeLastError() == 0


def test_module_load_and_launch_generated_kernel(rt, pkg, oracle, rng):
    """The call sequence the lowering emits for a generated kernel:
    mgpuModuleFileLoad -> mgpuModuleGetFunction(name) -> mgpuLaunchKernel with an
    array of pointers to bare-pointer arguments, two streams joined by events."""
    rt.mgpuModuleFileLoad(pkg.OPS_MODULE.encode())
    fn = rt.mgpuModuleGetFunction(b"main_graph_kernel")
    assert fn
    n = 3 * 640 * 640
    a = rng.uniform(-1, 1, n).astype(np.float32)
    b = rng.uniform(-1, 1, n).astype(np.float32)
    c = np.zeros(n, np.float32)
    data, kern = rt.mgpuStreamCreate(), rt.mgpuStreamCreate()
    ev_d, ev_k = rt.mgpuEventCreateWithStream(data), rt.mgpuEventCreate()
    da, db, dc = (rt.mgpuMemAlloc(n * 4, data) for _ in range(3))
    rt.mgpuMemcpy(da, host_ptr(a), n * 4, data)
    rt.mgpuMemcpy(db, host_ptr(b), n * 4, data)
    rt.mgpuEventRecord(ev_d, data)
    rt.mgpuStreamWaitEvent(kern, ev_d)
    args = [ctypes.c_void_p(da), ctypes.c_void_p(db), ctypes.c_void_p(dc), ctypes.c_int64(n)]
    params = (ctypes.c_void_p * 4)(*[ctypes.cast(ctypes.pointer(x), ctypes.c_void_p) for x in args])
    rt.mgpuLaunchKernel(fn, 1200, 1, 1, 256, 1, 1, 0, kern, params, None)
    rt.mgpuEventRecord(ev_k, kern)
    rt.mgpuStreamWaitEvent(data, ev_k)
    rt.mgpuMemcpy(host_ptr(c), dc, n * 4, data)
    rt.mgpuStreamSynchronize(data)
    assert np.array_equal(c.view(np.uint32), oracle.add_f32(a, b).view(np.uint32))
    for p in (da, db, dc):
        rt.mgpuMemFree(p, data)
    rt.mgpuEventDestroy(ev_d)
    rt.mgpuEventDestroy(ev_k)
    rt.mgpuStreamDestroy(data)
    rt.mgpuStreamDestroy(kern)
    rt.mgpuModuleUnload()
    assert rt.mgpuRuntimeTakeLastError() == 0


def test_event_timing(rt):
    s = rt.mgpuStreamCreate()
    e0, e1 = rt.mgpuEventEnableTimeCreate(), rt.mgpuEventEnableTimeCreate()
    d = rt.mgpuMemAlloc(64 << 20, s)
    rt.mgpuEventRecord(e0, s)
    for _ in range(4):
        rt.mgpuMemset32(d, 1, 16 << 20, s)
    rt.mgpuEventRecord(e1, s)
    rt.mgpuEventSynchronize(e1)
    ms = rt.mgpuEventElapsedTime(e0, e1)
    assert 0 < ms < 1000
    rt.mgpuMemFree(d, s)
    rt.mgpuEventDestroy(e0)
    rt.mgpuEventDestroy(e1)
    rt.mgpuStreamDestroy(s)


def test_errors_are_reported_not_fatal(rt, capfd):
    """Print-and-continue convention: a failing call writes
    '<expr>' failed with '<name>' to stderr and returns."""
    rt.mgpuRuntimeTakeLastError()
    rt.mgpuModuleFileLoad(b"/nonexistent/ops.hsaco")
    err = capfd.readouterr().err
    assert "failed with" in err and "hipModuleLoad" in err
    assert rt.mgpuRuntimeTakeLastError() != 0
    assert rt.mgpuRuntimeTakeLastError() == 0
    assert not rt.mgpuModuleGetFunction(b"main_graph_kernel")  # no module loaded
    rt.mgpuRuntimeTakeLastError()
    rt.mgpuLaunchKernel(None, 1, 1, 1, 64, 1, 1, 0, None, None, None)
    assert rt.mgpuRuntimeTakeLastError() != 0
    capfd.readouterr()


def _runner(pkg, name):
    return os.path.join(pkg.BIN_DIR, name)


def test_gpu_runner_add_model_matches_cpu_runner(pkg, gpu, tmp_path, oracle):
    a = gen_data.gen_data("3_640_640", seed=20240, dist="uniform")
    b = gen_data.gen_data("3_640_640", seed=20241, dist="uniform")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    outs = {}
    for dev in ("gpu", "cpu"):
        out = str(tmp_path / f"c_{dev}.dat")
        cmd = [_runner(pkg, f"multi-device-{dev}-runner"), os.path.join(pkg.LIB_DIR, "models", f"add_{dev}.so"),
               "--data", f"{fa},{fb}", "--out-data", out, "--rerun", "3"]
        if dev == "gpu":
            cmd += ["--ops", pkg.OPS_MODULE]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr
        assert "Run \t3\ttimes" in r.stdout and "Average time:\t" in r.stdout
        outs[dev] = np.fromfile(out, np.float32)
    assert np.array_equal(outs["gpu"].view(np.uint32), outs["cpu"].view(np.uint32))
    assert np.array_equal(outs["gpu"].view(np.uint32), oracle.add_f32(a, b).reshape(-1).view(np.uint32))


def test_gpu_runner_runs_what_lib_generate_emitted(pkg, gpu, tmp_path, oracle):
    """The add model and its kernel module after multi-device-lib-generate took
    them from LLVM IR (host: opt -> llc -> .so, kernel: AMDGPU IR -> ops.hsaco)."""
    gen = os.path.join(pkg.LIB_DIR, "models", "generated")
    a = gen_data.gen_data("3_640_640", seed=31, dist="uniform")
    b = gen_data.gen_data("3_640_640", seed=32, dist="uniform")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    out = str(tmp_path / "c.dat")
    r = subprocess.run([_runner(pkg, "multi-device-gpu-runner"), os.path.join(gen, "add_gpu.so"), "--ops",
                        os.path.join(gen, "ops.hsaco"), "--data", f"{fa},{fb}", "--out-data", out],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, np.float32).view(np.uint32), oracle.add_f32(a, b).reshape(-1).view(np.uint32))

def test_gpu_runner_layernorm_and_fmha_models(pkg, gpu, tmp_path, oracle):
    x = gen_data.gen_data("32_128_768", seed=1, dist="normal")
    g = gen_data.gen_data("768", seed=2, dist="normal", mean=1.0, std=0.02)
    b = gen_data.gen_data("768", seed=3, dist="normal", std=0.02)
    files = [gen_data.save_data(t, str(tmp_path / n)) for t, n in ((x, "x"), (g, "g"), (b, "b"))]
    out = str(tmp_path / "y.dat")
    r = subprocess.run([_runner(pkg, "multi-device-gpu-runner"), os.path.join(pkg.LIB_DIR, "models", "layernorm_gpu.so"),
                        "--ops", pkg.OPS_MODULE, "--input", "32_128_768,768,768", "--output", "32_128_768",
                        "--data", ",".join(files), "--out-data", out], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    y = np.fromfile(out, np.float32).reshape(x.shape)
    ref = oracle.layernorm(x, g, b)
    assert np.all(np.abs(y - ref) <= 1e-5 * np.abs(ref) + 1e-6)

    qkv = (gen_data.gen_data("4_128_3_12_64", seed=4, dist="normal") / 8).astype(np.float16)
    fq = gen_data.save_data(qkv, str(tmp_path / "qkv"))
    out = str(tmp_path / "o.dat")
    r = subprocess.run([_runner(pkg, "multi-device-gpu-runner"), os.path.join(pkg.LIB_DIR, "models", "fmha_gpu.so"),
                        "--ops", pkg.OPS_MODULE, "--dtype", "f16", "--input", "4_128_3_12_64", "--output",
                        "4_128_768", "--data", fq, "--out-data", out, "--rerun", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    o = np.fromfile(out, np.float16).reshape(4, 128, 768).astype(np.float32)
    assert np.abs(o - oracle.fmha(qkv)).max() <= 2e-3
