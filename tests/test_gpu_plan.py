"""Device plans executed on the GPU by multi-device-gpu-runner: the lowered
call list (two streams, events, device buffers, C-ABI op calls) run for real,
results against the oracle at the tolerances of the op tests."""
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

PKG = os.path.join(ROOT, "multi-device-model-compiler_amd")
PLANS = os.path.join(PKG, "plans")
sys.path.insert(0, os.path.join(PKG, "tools"))
import gen_data  # noqa: E402


def run_plan(pkg, plan, arrays, out_dtype, out_shape, tmp_path, extra=()):
    files = []
    for i, a in enumerate(arrays):
        f = str(tmp_path / f"in{i}.dat")
        np.ascontiguousarray(a).tofile(f)
        files.append(f)
    out = str(tmp_path / "out.dat")
    cmd = [os.path.join(pkg.BIN_DIR, "multi-device-gpu-runner"), str(plan), "--ops", pkg.OPS_MODULE,
           "--out-data", out, *extra]
    if files:
        cmd += ["--data", ",".join(files)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "failed with" not in r.stderr and "mgpu" not in r.stderr, r.stderr
    return np.fromfile(out, out_dtype).reshape(out_shape), r


def test_add_plans_library_op_and_generated_kernel(pkg, gpu, tmp_path, oracle):
    a = gen_data.gen_data("3_640_640", seed=20240, dist="uniform")
    b = gen_data.gen_data("3_640_640", seed=20241, dist="uniform")
    ref = oracle.add_f32(a, b).view(np.uint32)
    for name in ("add.plan", "add_generated_kernel.plan"):
        c, r = run_plan(pkg, os.path.join(PLANS, name), [a, b], np.float32, a.shape, tmp_path, ("--rerun", "3"))
        assert np.array_equal(c.view(np.uint32), ref), name
        assert "Run \t3\ttimes" in r.stdout and "Average time:\t" in r.stdout


def test_layernorm_and_attention_plans_at_config_size(pkg, gpu, tmp_path, oracle):
    x = gen_data.gen_data("32_128_768", seed=1, dist="normal")
    g = gen_data.gen_data("768", seed=2, dist="normal", mean=1.0, std=0.02)
    b = gen_data.gen_data("768", seed=3, dist="normal", std=0.02)
    y, _ = run_plan(pkg, os.path.join(PLANS, "layernorm.plan"), [x, g, b], np.float32, x.shape, tmp_path)
    ref = oracle.layernorm(x, g, b)
    assert np.all(np.abs(y - ref) <= 1e-5 * np.abs(ref) + 1e-6)

    qkv = gen_data.gen_data("32_128_3_12_64", seed=4, dist="normal").astype(np.float16)
    o, _ = run_plan(pkg, os.path.join(PLANS, "fmha.plan"), [qkv], np.float16, (32, 128, 768), tmp_path)
    ref = oracle.fmha(qkv)
    assert np.all(np.abs(o.astype(np.float32) - ref) <= 2e-3 * np.maximum(1.0, np.abs(ref)))


def layer_tol(ref):
    return 5e-3 + 4e-3 * np.abs(ref)  # see tests/test_gpu_ops_misc.py


def test_bert_layer_composed_from_primitive_ops(pkg, gpu, tmp_path, oracle):
    """The shipped BERT-base layer plan at batch 4: six library calls chained on
    device buffers, weights uploaded from the raw files next to the plan.
    Post-LN ordering and erf-GELU come from the benchmark configuration, not
    from the reference's layer (pre-LN / ReLU / causal)."""
    rng = np.random.Generator(np.random.PCG64(77))
    B, S, d, ffn, H = 4, 128, 768, 3072, 12
    text = open(os.path.join(PLANS, "bert_layer.plan")).read().replace("32x128x", f"{B}x{S}x")
    plan = tmp_path / "bert_layer.plan"
    plan.write_text(text)
    h16 = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float16)
    gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
    names = ["wqkv", "bqkv", "wo", "bo", "gamma1", "beta1", "w1", "b1", "w2", "b2", "gamma2", "beta2"]
    P = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
         h16(d), gam(), h16(d)]
    for n, p in zip(names, P):
        p.tofile(str(tmp_path / f"{n}.dat"))
    x = rng.standard_normal((B, S, d)).astype(np.float16)
    got, _ = run_plan(pkg, plan, [x], np.float16, (B, S, d), tmp_path, ("--rerun", "2"))
    ref = oracle.bert_layer_f16(x, *P, heads=H)
    err = np.abs(got.astype(np.float32) - ref)
    assert np.all(err <= layer_tol(ref)), err.max()
    assert err.mean() <= 5e-4
    # the same plan through the CPU lowering and the CPU op library
    cpu_out = str(tmp_path / "out_cpu.dat")
    r = subprocess.run([os.path.join(pkg.BIN_DIR, "multi-device-cpu-runner"), str(plan), "--data", str(tmp_path / "in0.dat"),
                        "--out-data", cpu_out], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    cpu = np.fromfile(cpu_out, np.float16).reshape(B, S, d).astype(np.float32)
    diff = np.abs(got.astype(np.float32) - cpu)
    assert np.all(diff <= layer_tol(cpu)), diff.max()
    assert diff.mean() <= 5e-4


def test_multi_head_attention_layer_op(pkg, gpu, tmp_path, oracle):
    """device.multi-head-attention-layer (DeviceOps.td:145-183) lowers to
    mgpuLLMDecodingContextLayer with the argument order of
    ConvertDeviceToLLVM.cpp:741-748."""
    rng = np.random.Generator(np.random.PCG64(78))
    B, S, d, ffn, H = 2, 128, 512, 2048, 8
    f = lambda *s, sc=0.03: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    plan = tmp_path / "layer.plan"
    plan.write_text(
        f"func @main_graph(%x: {B}x{S}x{d}xf32, %qkv: {d}x{3 * d}xf32, %aw: {d}x{d}xf32, %ab: {d}xf32, "
        f"%f1w: {d}x{ffn}xf32, %f1b: {ffn}xf32, %f2w: {ffn}x{d}xf32, %f2b: {d}xf32) -> (%y: {B}x{S}x{d}xf32) {{\n"
        f"  %y = device.multi-head-attention-layer %x, %qkv, %aw, %ab, %f1w, %f1b, %f2w, %f2b "
        f"{{head_num = {H}, norm_first = true, is_casual = true, act = \"relu\", batch = {B}, seq_len = {S}}} : {B}x{S}x{d}xf32\n"
        "  return\n}\n")
    got, _ = run_plan(pkg, plan, [x] + W, np.float32, (B, S, d), tmp_path)
    ref = oracle.decoding_context_layer(x, *W, heads=H, causal=True, act=oracle.ACT_RELU)
    assert np.all(np.abs(got - ref) <= layer_tol(ref))


def test_resnet_block_plan(pkg, gpu, tmp_path, oracle):
    """conv + ReLU, conv + shortcut + ReLU, max pool: device.conv2d / device.pool2d through
    mgpuConv2d / mgpuPool2d, the shortcut operand staying on the device across two ops."""
    rng = np.random.Generator(np.random.PCG64(79))
    c = 64
    plan = tmp_path / "resnet_block.plan"
    plan.write_text(open(os.path.join(PLANS, "resnet_block.plan")).read())
    w1, w2 = [(rng.standard_normal((c, c, 3, 3)) / 24).astype(np.float32) for _ in range(2)]
    b1, b2 = [rng.standard_normal(c).astype(np.float32) for _ in range(2)]
    for name, a in (("w1", w1), ("b1", b1), ("w2", w2), ("b2", b2)):
        a.tofile(str(tmp_path / f"{name}.dat"))
    x = rng.standard_normal((4, c, 28, 28)).astype(np.float32)
    y, _ = run_plan(pkg, plan, [x], np.float32, (4, c, 14, 14), tmp_path)
    h = oracle.conv2d(x, w1, b1, None, (1, 1, 1, 1), relu=True)
    r = oracle.conv2d(h, w2, b2, x, (1, 1, 1, 1), relu=True)
    ref = oracle.pool2d(r, (2, 2), stride=(2, 2))
    assert np.all(np.abs(y - ref) <= 4e-3 * (1.0 + np.abs(ref)))


def test_bf16_pipeline_cast_matmul_cast(pkg, gpu, tmp_path, oracle, rng):
    """fp32 in -> bf16 cast -> bf16 GEMM with bias and ReLU -> fp32 out: the
    bf16 entry points reached through the plan lowering."""
    M, K, N = 64, 128, 96
    body = f"""func @main_graph(%x: {M}x{K}xf32, %w: {K}x{N}xf32, %b: {N}xf32) -> (%y: {M}x{N}xf32) {{
  %xh = device.cast %x : {M}x{K}xbf16
  %wh = device.cast %w : {K}x{N}xbf16
  %bh = device.cast %b : {N}xbf16
  %yh = device.matmul-ex %xh, %wh, %bh, none {{act = "relu"}} : {M}x{N}xbf16
  %y = device.cast %yh : {M}x{N}xf32
  return
}}
"""
    plan = tmp_path / "bf16.plan"
    plan.write_text(body)
    lower = subprocess.run([os.path.join(pkg.BIN_DIR, "multi-device-plan-lower"), str(plan)], capture_output=True, text=True)
    assert lower.returncode == 0, lower.stderr
    for callee in ("mgpuCastF32ToBF16", "mgpuMatmulExBF16", "mgpuCastBF16ToF32"):
        assert callee in lower.stdout
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    y, _ = run_plan(pkg, plan, [x, w, b], np.float32, (M, N), tmp_path)
    ref = oracle.gemm(oracle.float_to_bf16(x), oracle.float_to_bf16(w), oracle.float_to_bf16(b), act=oracle.ACT_RELU, bf16=True)
    tol = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -14))) - 7) + 4e-3
    assert np.all(np.abs(y - ref) <= tol), np.abs(y - ref).max()
