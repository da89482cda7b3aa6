"""Device plan -> runtime-call lowering (C++, no GPU): the call sequence the
reference's DeviceDataCopyGeneration + AsyncDependencyConvert +
ConvertDeviceToLLVM passes produce for a function of device ops - two streams
with one event each, uploads / allocations / frees on the data stream, ops on
the kernel stream, a record + wait for every cross-stream edge, the closing
wait - plus the plan verifier and the plan-driven CPU runner."""
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT

PKG = os.path.join(ROOT, "multi-device-model-compiler_amd")
LOWER = os.path.join(PKG, "bin", "multi-device-plan-lower")
CPU_RUNNER = os.path.join(PKG, "bin", "multi-device-cpu-runner")
PLANS = os.path.join(PKG, "plans")


def lower(path, *flags):
    return subprocess.run([LOWER, path, *flags], capture_output=True, text=True, timeout=60)


def lower_text(tmp_path, text, *flags):
    f = tmp_path / "t.plan"
    f.write_text(text)
    return lower(str(f), *flags)


ADD_CALLS = """\
%DataStream = mgpuStreamCreate()
%DataEvent = mgpuEventCreateWithStream(%DataStream)
%KernelStream = mgpuStreamCreate()
%KernelEvent = mgpuEventCreateWithStream(%KernelStream)
// device.add (line 4)
%d0 = mgpuMemAlloc(4915200, %DataStream)
mgpuMemcpy(%d0, %a, 4915200, %DataStream)
%d1 = mgpuMemAlloc(4915200, %DataStream)
mgpuMemcpy(%d1, %b, 4915200, %DataStream)
%d2 = mgpuMemAlloc(4915200, %DataStream)
mgpuEventRecord(%DataEvent, %DataStream)
mgpuStreamWaitEvent(%KernelStream, %DataEvent)
mgpuAddF32(%d0, %d1, %d2, 1228800, %KernelStream)
mgpuEventRecord(%KernelEvent, %KernelStream)
mgpuStreamWaitEvent(%DataStream, %KernelEvent)
mgpuMemFree(%d0, %DataStream)
mgpuMemFree(%d1, %DataStream)
mgpuMemcpy(%c, %d2, 4915200, %DataStream)
mgpuMemFree(%d2, %DataStream)
mgpuEventDestroy(%DataEvent)
mgpuStreamSynchronize(%DataStream)
mgpuStreamDestroy(%DataStream)
mgpuEventDestroy(%KernelEvent)
mgpuStreamSynchronize(%KernelStream)
mgpuStreamDestroy(%KernelStream)
"""


def test_add_plan_lowers_to_the_reference_call_sequence():
    """The hand-lowered add model (csrc/models/add_gpu.cpp) and this listing
    are the same sequence: stream + event creation per stream
    (ConvertDeviceToLLVM.cpp:358-372), allocations and copies on the data
    stream, record/wait before the op (AsyncDependencyConvert.cpp:89-96), the
    op with the stream as last argument, record/wait back before the data
    stream touches the buffers again, event destroy / synchronize / destroy
    per stream (ConvertDeviceToLLVM.cpp:345-354)."""
    r = lower(os.path.join(PLANS, "add.plan"))
    assert r.returncode == 0, r.stderr
    assert r.stdout == ADD_CALLS


def test_generated_kernel_launch_uses_the_bare_pointer_convention():
    r = lower(os.path.join(PLANS, "add_generated_kernel.plan"))
    assert r.returncode == 0, r.stderr
    assert '%d3 = mgpuModuleGetFunction("main_graph_kernel")' in r.stdout
    assert ("mgpuLaunchKernel(%d3, 1200, 1, 1, 256, 1, 1, 0 : i32, %KernelStream, "
            "[&%d0, &%d1, &%d2, &1228800], null)") in r.stdout


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(PLANS) if f.endswith(".plan")))
def test_every_shipped_plan_keeps_the_two_stream_discipline(name):
    r = lower(os.path.join(PLANS, name))
    assert r.returncode == 0, r.stderr  # includes the ordering check of the call list
    lines = [l for l in r.stdout.splitlines() if not l.startswith("//")]
    assert lines[:4] == ADD_CALLS.splitlines()[:4] and lines[-6:] == ADD_CALLS.splitlines()[-6:]
    prev2 = None
    for i, l in enumerate(lines[4:-6], 4):
        callee = l.split("(")[0].split("= ")[-1]
        if callee in ("mgpuMemAlloc", "mgpuMemcpy", "mgpuMemFree"):
            assert l.endswith("%DataStream)"), l
        elif callee in ("mgpuEventRecord", "mgpuStreamWaitEvent", "mgpuModuleGetFunction"):
            pass
        else:  # an op: on the kernel stream, right behind a data -> kernel record + wait
            assert "%KernelStream" in l, l
            k = i - 1 if "mgpuModuleGetFunction" not in lines[i - 1] else i - 2
            assert lines[k] == "mgpuStreamWaitEvent(%KernelStream, %DataEvent)"
            assert lines[k - 1] == "mgpuEventRecord(%DataEvent, %DataStream)"
    # every allocation is freed exactly once
    allocs = [l.split(" = ")[0] for l in lines if "mgpuMemAlloc" in l]
    frees = [l.split("(")[1].split(",")[0] for l in lines if l.startswith("mgpuMemFree")]
    assert sorted(allocs) == sorted(frees)


def test_bert_layer_plan_keeps_values_on_the_device_and_views_share_a_buffer():
    r = lower(os.path.join(PLANS, "bert_layer.plan"))
    assert r.returncode == 0, r.stderr
    out = r.stdout
    # one upload per host value (input + 12 weights), one copy back
    assert out.count("mgpuMemcpy(") == 14
    # the reshape makes no call: attention reads the buffer the QKV GEMM wrote
    assert "mgpuMatmulExF16(%d0, %d1, %d2, %d3, null, 4096, 2304, 768, 1 : i32, 0 : i32, 0 : i32, %KernelStream)" in out
    assert "mgpuFusedMHAF16(%d3, null, %d4, 32 : i32, 128 : i32, 12 : i32, 64 : i32, 0.125 : f32, 0 : i32, %KernelStream)" in out
    assert "device.reshape" not in out
    # GELU rides on the activation code of the FFN1 GEMM
    assert "4096, 3072, 768, 1 : i32, 2 : i32, 0 : i32, %KernelStream)" in out


def test_conv_and_pool_lower_with_the_reference_argument_order():
    """ConvertDeviceToLLVM.cpp:533-548,612-627: pointers, then N IC H W OC KH KW OH OW, PHL PWL PHR PWR,
    SH SW, DH DW, hasPostAdd, containRelu, stream; pool: N C H W OH OW KH KW PHL PWL PHR PWR SH SW method."""
    r = lower(os.path.join(PLANS, "resnet_block.plan"))
    assert r.returncode == 0, r.stderr
    assert ("mgpuConv2d(%d0, %d1, %d2, %d3, null, 4, 64, 28, 28, 64, 3, 3, 28, 28, 1, 1, 1, 1, 1, 1, 1, 1, "
            "false, true, %KernelStream)") in r.stdout
    assert ("mgpuConv2d(%d3, %d4, %d5, %d6, %d0, 4, 64, 28, 28, 64, 3, 3, 28, 28, 1, 1, 1, 1, 1, 1, 1, 1, "
            "true, true, %KernelStream)") in r.stdout
    assert "mgpuPool2d(%d6, %d7, 4, 64, 28, 28, 14, 14, 2, 2, 0, 0, 0, 0, 2, 2, 0, %KernelStream)" in r.stdout
    # the shortcut keeps %x on the device until the second convolution has read it
    lines = r.stdout.splitlines()
    assert lines.index("mgpuMemFree(%d0, %DataStream)") > [i for i, l in enumerate(lines) if "mgpuConv2d" in l][1]


def test_plan_round_trip(tmp_path):
    src = os.path.join(PLANS, "bert_layer.plan")
    printed = lower(src, "--emit", "plan")
    assert printed.returncode == 0
    again = lower_text(tmp_path, printed.stdout)
    assert again.returncode == 0, again.stderr
    strip = lambda s: [l for l in s.splitlines() if not l.startswith("//")]
    assert strip(again.stdout) == strip(lower(src).stdout)


HEAD = "func @main_graph(%x: 4x8xf32, %w: 8x16xf32, %b: 16xf32) -> (%y: 4x16xf32) {\n"


@pytest.mark.parametrize("body,message", [
    ("  %y = device.matmul %x, %w, %b : 4x16xf32\n  return\n", None),
    ("  %y = device.matmul %x, %w, %q : 4x16xf32\n  return\n}\n", "line 2: %q is used before its definition"),
    ("  %y = device.conv3d %x : 4x16xf32\n  return\n}\n", "line 2: device.conv3d: unknown op"),
    # MatmulOp::verify (DeviceDialect.cpp:66-100): K mismatch, bias length, output shape
    ("  %y = device.matmul %w, %w, %b : 4x16xf32\n  return\n}\n", "weight must be [K, N]"),
    ("  %y = device.matmul %x, %w, %x : 4x16xf32\n  return\n}\n", "bias must be 16xf32"),
    ("  %t = device.matmul %x, %w, %b : 4x8xf32\n  return\n}\n", "output must be [..., N]"),
    ("  %y = device.matmul %x, %w, %b : 4x16xf32\n  %y = device.matmul %x, %w, %b : 4x16xf32\n  return\n}\n",
     "line 3: function result %y is produced twice"),
    ("  %t = device.matmul %x, %w, %b : 4x16xf32\n  return\n}\n", "function result %y is never produced"),
    ("  %y = device.matmul %x, %w, %b : 4x16xf32\n}\n", "line 3: missing return"),
    ("  %y = device.matmul %x, %w, %b {fast = true} : 4x16xf32\n  return\n}\n", "unknown attribute fast"),
    ("  %y = device.matmul-ex %x, %w, %b, none {act = \"tanh\"} : 4x16xf32\n  return\n}\n", "act is"),
    ("  %y = device.matmul %x, %w, none : 4x16xf32\n  return\n}\n", "operand 2 cannot be none"),
    ("  %y = device.layernorm %x, %b, %b : 4x16xf32\n  return\n}\n", "gamma must be 8xf32"),
    ("  %y = device.matmul %x, %w, %b : 4x16xf16\n  return\n}\n", "has type 4x16xf32 in the signature"),
])
def test_verifier_messages(tmp_path, body, message):
    r = lower_text(tmp_path, HEAD + body + ("}\n" if message is None else ""))
    if message is None:
        assert r.returncode == 0, r.stderr
    else:
        assert r.returncode == 1 and message in r.stderr, r.stderr


def test_attention_and_launch_verifiers(tmp_path):
    bad = [
        ("func @f(%q: 2x16x3x4x36xf16) -> (%o: 2x16x144xf16) {\n  %o = device.fused-mha %q, none : 2x16x144xf16\n  return\n}\n",
         "head_dim must be a multiple of 8"),
        ("func @f(%q: 2x16x3x4x64xf32) -> (%o: 2x16x256xf32) {\n  %o = device.fused-mha %q, none : 2x16x256xf32\n  return\n}\n",
         "qkv must be f16 or bf16"),
        ("func @f(%q: 2x16x3x4x64xf16, %l: 3xi32) -> (%o: 2x16x256xf16) {\n  %o = device.fused-mha %q, %l : 2x16x256xf16\n  return\n}\n",
         "key lengths must be Bxi32"),
        ("func @f(%a: 8xf32) -> (%c: 8xf32) {\n  %c = gpu.launch_func %a {kernel = \"k\", blocks = [1, 1, 1], threads = [2048, 1, 1]} : 8xf32\n  return\n}\n",
         "more than 1024 threads per block"),
        ("func @f(%a: 8xf32) -> (%c: 8xf32) {\n  %c = gpu.launch_func %a {blocks = [1, 1, 1], threads = [64, 1, 1]} : 8xf32\n  return\n}\n",
         "needs {kernel"),
    ]
    for text, message in bad:
        r = lower_text(tmp_path, text)
        assert r.returncode == 1 and message in r.stderr, (message, r.stderr)


def test_call_list_checker(tmp_path):
    """checkRuntimeProgram rejects call lists that break the discipline; driven
    from a small C++ program because the API is C++."""
    exe = str(tmp_path / "check_program_test")
    subprocess.run(["g++", "-O1", "-std=c++17", "-I" + os.path.join(PKG, "include"),
                    os.path.join(ROOT, "tests", "cpp", "check_program_test.cpp"), "-o", exe,
                    "-L" + os.path.join(PKG, "lib"), "-lmdmc_conversion", "-Wl,-rpath," + os.path.join(PKG, "lib")],
                   check=True, timeout=120)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "FAIL" not in r.stdout, r.stdout


def run_cpu_plan(tmp_path, text, arrays, out_dtype, out_shape, extra=()):
    plan = tmp_path / "m.plan"
    plan.write_text(text)
    files = []
    for i, a in enumerate(arrays):
        f = str(tmp_path / f"in{i}.dat")
        np.ascontiguousarray(a).tofile(f)
        files.append(f)
    out = str(tmp_path / "out.dat")
    r = subprocess.run([CPU_RUNNER, str(plan), "--data", ",".join(files), "--out-data", out, *extra],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    return np.fromfile(out, out_dtype).reshape(out_shape), r


def test_cpu_runner_executes_plans(tmp_path, oracle, rng):
    """The CPU lowering calls the CPU op library on the host buffers
    (ConvertDeviceToLLVM.cpp:433-436); results against the oracle."""
    a = rng.uniform(-1, 1, (3, 64, 64)).astype(np.float32)
    b = rng.uniform(-1, 1, (3, 64, 64)).astype(np.float32)
    g = rng.standard_normal(64).astype(np.float32)
    be = rng.standard_normal(64).astype(np.float32)
    text = ("func @main_graph(%a: 3x64x64xf32, %b: 3x64x64xf32, %g: 64xf32, %be: 64xf32) -> (%y: 3x64x64xf32) {\n"
            "  %c = device.add %a, %b : 3x64x64xf32\n"
            "  %y = device.layernorm %c, %g, %be {eps = 1e-5} : 3x64x64xf32\n  return\n}\n")
    y, r = run_cpu_plan(tmp_path, text, [a, b, g, be], np.float32, a.shape, ("--rerun", "2"))
    ref = oracle.layernorm(oracle.add_f32(a, b), g, be)
    assert np.all(np.abs(y - ref) <= 1e-5 * np.abs(ref) + 2e-6)
    assert "Run \t2\ttimes" in r.stdout and "Average time:\t" in r.stdout

    x = rng.standard_normal((5, 24)).astype(np.float32)
    w = rng.standard_normal((24, 40)).astype(np.float32)
    bias = rng.standard_normal(40).astype(np.float32)
    text = ("func @main_graph(%x: 5x24xf32, %w: 24x40xf32, %b: 40xf32) -> (%y: 5x40xf32) {\n"
            "  %y = device.matmul %x, %w, %b : 5x40xf32\n  return\n}\n")
    y, _ = run_cpu_plan(tmp_path, text, [x, w, bias], np.float32, (5, 40))
    assert np.allclose(y, x.astype(np.float64) @ w + bias, rtol=1e-5, atol=1e-5)

    qkv = rng.standard_normal((2, 70, 3, 2, 64)).astype(np.float16)
    lens = np.array([70, 33], np.int32)
    text = ("func @main_graph(%q: 2x70x3x2x64xf16, %l: 2xi32) -> (%o: 2x70x128xf16) {\n"
            "  %o = device.fused-mha %q, %l {causal = true} : 2x70x128xf16\n  return\n}\n")
    o, _ = run_cpu_plan(tmp_path, text, [qkv, lens], np.float16, (2, 70, 128))
    ref = oracle.fmha(qkv, lens, causal=True)
    assert np.abs(o.astype(np.float32) - ref).max() <= 2e-3 * max(1.0, np.abs(ref).max())


def test_cpu_runner_executes_the_resnet_block(tmp_path, oracle, rng):
    text = open(os.path.join(PLANS, "resnet_block.plan")).read().replace(" 4x64x", " 2x64x")
    c = 64
    w1, w2 = [(rng.standard_normal((c, c, 3, 3)) / 24).astype(np.float32) for _ in range(2)]
    b1, b2 = [rng.standard_normal(c).astype(np.float32) for _ in range(2)]
    for name, a in (("w1", w1), ("b1", b1), ("w2", w2), ("b2", b2)):
        a.tofile(str(tmp_path / f"{name}.dat"))
    x = rng.standard_normal((2, c, 28, 28)).astype(np.float32)
    y, _ = run_cpu_plan(tmp_path, text, [x], np.float32, (2, c, 14, 14))
    h = oracle.conv2d(x, w1, b1, None, (1, 1, 1, 1), relu=True)
    r = oracle.conv2d(h, w2, b2, x, (1, 1, 1, 1), relu=True)
    ref = oracle.pool2d(r, (2, 2), stride=(2, 2))
    assert np.abs(y - ref).max() <= 1e-4


def test_conv_pool_verifier_messages(tmp_path):
    head = "func @f(%x: 1x2x8x8xf32, %w: 3x2x3x3xf32, %b: 3xf32) -> (%y: 1x3x8x8xf32) {\n"
    for body, message in [
        ("  %y = device.conv2d %x, %w, %b, none {pad = [1, 1, 1, 1]} : 1x3x8x8xf32\n  return\n}\n", None),
        ("  %y = device.conv2d %x, %w, %b, none : 1x3x8x8xf32\n  return\n}\n", "output size does not follow"),
        ("  %y = device.conv2d %x, %w, %x, none {pad = [1, 1, 1, 1]} : 1x3x8x8xf32\n  return\n}\n", "bias must be 3xf32"),
        ("  %y = device.conv2d %x, %w, %b, none {pad = [1, 1, 1, 1], kernel = [5, 5]} : 1x3x8x8xf32\n  return\n}\n",
         "kernel disagrees"),
        ("  %y = device.conv2d %w, %w, %b, none {pad = [1, 1, 1, 1]} : 1x3x8x8xf32\n  return\n}\n", "batch or channel counts"),
        ("  %t = device.pool2d %x {kernel = [2, 2], stride = [2, 2], method = \"min\"} : 1x2x4x4xf32\n  return\n}\n", "method is"),
        ("  %t = device.pool2d %x {kernel = [2, 2], stride = [2, 2], method = \"avg\"} : 1x2x5x4xf32\n  return\n}\n",
         "output size does not follow"),
    ]:
        r = lower_text(tmp_path, head + body)
        if message is None:
            assert r.returncode == 0, r.stderr
        else:
            assert r.returncode == 1 and message in r.stderr, (message, r.stderr)


def test_cpu_runner_reports_missing_lowerings_and_bad_files(tmp_path):
    bf16 = tmp_path / "bf16.plan"
    bf16.write_text("func @main_graph(%x: 4x8xf32) -> (%y: 4x8xbf16) {\n  %y = device.cast %x : 4x8xbf16\n  return\n}\n")
    r = subprocess.run([CPU_RUNNER, str(bf16)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "has no CPU lowering" in r.stderr
    short = tmp_path / "a.dat"
    short.write_bytes(b"\0" * 12)
    r = subprocess.run([CPU_RUNNER, os.path.join(PLANS, "add.plan"), "--data", f"{short},{short}"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "Wrong File size" in r.stderr
    r = subprocess.run([CPU_RUNNER, str(tmp_path / "missing.plan")], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "Failed to open plan" in r.stderr


def layer_tol(ref):
    return 5e-3 + 4e-3 * np.abs(ref)  # fp16 output after ~6 fp16-rounded stages, see tests/test_gpu_ops_misc.py


def test_cpu_runner_executes_the_bert_layer_plan(tmp_path, oracle):
    """plans/bert_layer.plan (six primitive calls: matmul-ex, fused-mha, add-residual-layernorm)
    through the CPU lowering and the CPU op library, at batch 2, against the oracle."""
    rng = np.random.Generator(np.random.PCG64(177))
    B, S, d, ffn, H = 2, 128, 768, 3072, 12
    text = open(os.path.join(PLANS, "bert_layer.plan")).read().replace("32x128x", f"{B}x{S}x")
    h16 = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float16)
    gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
    names = ["wqkv", "bqkv", "wo", "bo", "gamma1", "beta1", "w1", "b1", "w2", "b2", "gamma2", "beta2"]
    P = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
         h16(d), gam(), h16(d)]
    for n, p in zip(names, P):
        p.tofile(str(tmp_path / f"{n}.dat"))
    x = rng.standard_normal((B, S, d)).astype(np.float16)
    got, r = run_cpu_plan(tmp_path, text, [x], np.float16, (B, S, d), ("--rerun", "1"))
    assert "Average time:\t" in r.stdout
    ref = oracle.bert_layer_f16(x, *P, heads=H)
    err = np.abs(got.astype(np.float32) - ref)
    assert np.all(err <= layer_tol(ref)), err.max()
    assert err.mean() <= 5e-4


def test_cpu_runner_executes_the_layer_ops(tmp_path, oracle):
    """device.multi-head-attention-layer -> mcpuLLMDecodingContextLayer (the reference's CPU
    signature, Kernels/CPU/Ops.h:38-43) and device.bert-encoder-layer -> mcpuBertEncoderLayerF16."""
    rng = np.random.Generator(np.random.PCG64(178))
    B, S, d, ffn, H = 2, 64, 256, 512, 4
    f = lambda *s, sc=0.03: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    text = (f"func @main_graph(%x: {B}x{S}x{d}xf32, %qkv: {d}x{3 * d}xf32, %aw: {d}x{d}xf32, %ab: {d}xf32, "
            f"%f1w: {d}x{ffn}xf32, %f1b: {ffn}xf32, %f2w: {ffn}x{d}xf32, %f2b: {d}xf32) -> (%y: {B}x{S}x{d}xf32) {{\n"
            f"  %y = device.multi-head-attention-layer %x, %qkv, %aw, %ab, %f1w, %f1b, %f2w, %f2b "
            f"{{head_num = {H}, norm_first = true, is_casual = true, act = \"relu\", batch = {B}, seq_len = {S}}} : {B}x{S}x{d}xf32\n"
            "  return\n}\n")
    got, _ = run_cpu_plan(tmp_path, text, [x] + W, np.float32, (B, S, d))
    ref = oracle.decoding_context_layer(x, *W, heads=H, causal=True, act=oracle.ACT_RELU)
    assert np.all(np.abs(got - ref) <= layer_tol(ref)), np.abs(got - ref).max()
    assert np.array_equal(got, got.astype(np.float16).astype(np.float32))  # the final cast comes from fp16
    got, _ = run_cpu_plan(tmp_path, text.replace("norm_first = true", "norm_first = false"), [x] + W, np.float32,
                          (B, S, d))
    ref = oracle.decoding_context_layer(x, *W, heads=H, causal=True, act=oracle.ACT_RELU, norm_first=False)
    assert np.all(np.abs(got - ref) <= layer_tol(ref)), np.abs(got - ref).max()  # post-LN ordering

    h16 = lambda *s: (0.05 * rng.standard_normal(s)).astype(np.float16)
    gam = lambda: (1 + 0.05 * rng.standard_normal(d)).astype(np.float16)
    P = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
         h16(d), gam(), h16(d)]
    xh = rng.standard_normal((B, S, d)).astype(np.float16)
    lens = np.array([S, 17], np.int32)
    shapes = [f"{d}x{3 * d}", f"{3 * d}", f"{d}x{d}", f"{d}", f"{d}", f"{d}", f"{d}x{ffn}", f"{ffn}", f"{ffn}x{d}",
              f"{d}", f"{d}", f"{d}"]
    args = ", ".join(f"%p{i}: {sh}xf16" for i, sh in enumerate(shapes))
    text = (f"func @main_graph(%x: {B}x{S}x{d}xf16, {args}, %l: {B}xi32) -> (%y: {B}x{S}x{d}xf16) {{\n"
            f"  %y = device.bert-encoder-layer %x, {', '.join(f'%p{i}' for i in range(12))}, %l {{head_num = {H}, eps = 1e-5}} "
            f": {B}x{S}x{d}xf16\n  return\n}}\n")
    got, _ = run_cpu_plan(tmp_path, text, [xh] + P + [lens], np.float16, (B, S, d))
    ref = oracle.bert_layer_f16(xh, *P, heads=H, seqlens=lens)
    err = np.abs(got.astype(np.float32) - ref)
    assert np.all(err <= layer_tol(ref)), err.max()


def test_cpu_twins_of_the_16_bit_entry_points(oracle, rng):
    """mcpuLayerNormF16, mcpuAddResidualPreLayerNormF16/F32, mcpuMatmulExF16/F32 and the casts, called
    through ctypes, against the oracle at the bounds of their GPU counterparts."""
    import ctypes
    lib = ctypes.CDLL(os.path.join(PKG, "lib", "libmcpu_ops.so"))
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    m, n = 37, 200
    x = rng.standard_normal((m, n)).astype(np.float16)
    res = rng.standard_normal((m, n)).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(n)).astype(np.float16)
    b = (0.1 * rng.standard_normal(n)).astype(np.float16)
    y = np.empty_like(x)
    lib.mcpuLayerNormF16(ptr(x), ptr(g), ptr(b), ptr(y), ctypes.c_float(1e-5), m, n)
    ref = oracle.layernorm(x, g, b)
    ulp = lambda r: 2.0 ** (np.floor(np.log2(np.maximum(np.abs(r), 2.0 ** -14))) - 10)
    assert np.all(np.abs(y.astype(np.float32) - ref) <= ulp(ref) + 2e-6)
    s_out, y2 = np.empty_like(x), np.empty_like(x)
    lib.mcpuAddResidualPreLayerNormF16(ptr(x), ptr(res), ptr(g), ptr(b), ptr(s_out), ptr(y2), ctypes.c_float(1e-5), m, n)
    s_ref, y_ref = oracle.add_residual_layernorm(x, res, g, b)
    assert np.array_equal(s_out.astype(np.float32), oracle.half_to_float(oracle.cast_f32_to_f16(s_ref).view(np.uint16)).reshape(m, n))
    assert np.all(np.abs(y2.astype(np.float32) - y_ref) <= ulp(y_ref) + 2e-6)

    M, K, N = 45, 96, 72
    a = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    r16 = rng.standard_normal((M, N)).astype(np.float16)
    out = np.empty((M, N), np.float16)
    for act, residual in ((0, None), (1, None), (2, None), (0, r16)):
        lib.mcpuMatmulExF16(ptr(a), ptr(w), ptr(bias), ptr(out), ptr(residual) if residual is not None else None,
                            ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K), 1, act, int(residual is not None))
        ref = oracle.gemm(a, w, bias, residual, act=act)
        assert np.all(np.abs(out.astype(np.float32) - ref) <= ulp(ref) + 1e-5), (act, np.abs(out.astype(np.float32) - ref).max())
    a32, w32, b32 = a.astype(np.float32), w.astype(np.float32), bias.astype(np.float32)
    o32 = np.empty((M, N), np.float32)
    lib.mcpuMatmulExF32(ptr(a32), ptr(w32), ptr(b32), ptr(o32), None, ctypes.c_int64(M), ctypes.c_int64(N),
                        ctypes.c_int64(K), 1, 0, 0)
    assert np.allclose(o32, a32.astype(np.float64) @ w32 + b32, rtol=1e-5, atol=1e-5)

    f = np.concatenate([rng.standard_normal(1000) * 100, [0.0, -0.0, np.inf, -np.inf, 65504.0, 65520.0, 1e-8, 6e-8]]).astype(np.float32)
    h = np.empty(f.shape, np.float16)
    lib.mcpuCastF32ToF16(ptr(h), ptr(f), ctypes.c_size_t(f.size))
    assert np.array_equal(h.view(np.uint16), oracle.cast_f32_to_f16(f).view(np.uint16))
    back = np.empty(f.shape, np.float32)
    lib.mcpuCastF16ToF32(ptr(back), ptr(h), ctypes.c_size_t(f.size))
    assert np.array_equal(back.view(np.uint32), h.astype(np.float32).view(np.uint32))
