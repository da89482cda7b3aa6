"""Host runtime and CPU runner (C++): shape grammar, outputs-first parameter
order, raw file I/O, timing-line format and the non-fatal error messages of
the reference's lib/Runtime (RuntimeUtil.cpp, ModelInfo.cpp) and
tools/multi-device-cpu-runner.  Runs without a GPU."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT

TOOLS = os.path.join(ROOT, "multi-device-model-compiler_amd", "tools")
sys.path.insert(0, TOOLS)
import data_diff  # noqa: E402
import gen_data  # noqa: E402


@pytest.fixture(scope="module")
def paths(pkg):
    return {"cpu_runner": os.path.join(pkg.BIN_DIR, "multi-device-cpu-runner"),
            "gpu_runner": os.path.join(pkg.BIN_DIR, "multi-device-gpu-runner"),
            "models": os.path.join(pkg.LIB_DIR, "models")}


def run(cmd, **kw):
    return subprocess.run(cmd, capture_output=True, text=True, timeout=120, **kw)


def test_gen_data_is_seeded_and_named_like_the_reference(tmp_path):
    a = gen_data.gen_data("3_4_5", "f32", seed=3, dist="uniform")
    b = gen_data.gen_data("3_4_5", "f32", seed=3, dist="uniform")
    assert a.dtype == np.float32 and a.shape == (3, 4, 5) and np.array_equal(a, b)
    assert a.min() >= -1 and a.max() < 1
    r = gen_data.gen_data("8", "f32", seed=1, dist="random")
    assert r.min() >= 0 and r.max() < 1
    name = gen_data.save_data(a, str(tmp_path / "x"))
    assert name.endswith("x_float32_3_4_5.dat")
    assert np.array_equal(gen_data.load_data(name, "3_4_5"), a)
    assert np.array_equal(gen_data.load_data_raw(name), a.reshape(-1))


def test_data_diff_blocks(tmp_path, capsys):
    a = np.array([1.0, 2.0, 0.0, -4.0], np.float32)
    b = np.array([1.0, 2.5, 1e-3, -4.0], np.float32)
    fa, fb = str(tmp_path / "a.dat"), str(tmp_path / "b.dat")
    a.tofile(fa)
    b.tofile(fb)
    st = data_diff.data_diff(fa, fb)
    out = capsys.readouterr().out.splitlines()
    assert out[0].startswith("Absolute diff:\tMin:0.0\tMax:0.5\tMean:")
    assert out[1].startswith("Relative diff:\tMin:0.0\tMax:")
    assert out[2:] == ["Bound 1:\t0", "Bound 0.1:\t1", "Bound 0.01:\t1", "Bound 0.001:\t1",
                       "Bound 0.0001:\t2", "Bound 1e-05:\t2", "Bound 1e-06:\t2", "Bound 1e-07:\t2"]
    # relative diff uses |standard| + 1e-10 in the denominator
    assert st["rel"][1] == pytest.approx(1e-3 / 1e-10, rel=1e-3)


def test_cpu_runner_add_model_end_to_end(paths, tmp_path, oracle):
    a = gen_data.gen_data("3_640_640", seed=11, dist="uniform")
    b = gen_data.gen_data("3_640_640", seed=12, dist="uniform")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    out = str(tmp_path / "c.dat")
    r = run([paths["cpu_runner"], os.path.join(paths["models"], "add_cpu.so"), "--data", f"{fa},{fb}",
             "--out-data", out, "--rerun", "3"])
    assert r.returncode == 0, r.stderr
    c = np.fromfile(out, np.float32).reshape(3, 640, 640)
    assert np.array_equal(c.view(np.uint32), oracle.add_f32(a, b).view(np.uint32))
    lines = r.stdout.splitlines()
    assert lines[0] == "Run \t3\ttimes"
    assert re.fullmatch(r"Average time:\t[0-9.e+-]+\tseconds", lines[1])


def test_cpu_runner_other_shapes_and_flag_spellings(paths, tmp_path):
    a = gen_data.gen_data("2_3_5", seed=1, dist="normal")
    b = gen_data.gen_data("2_3_5", seed=2, dist="normal")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    out = str(tmp_path / "c.dat")
    r = run([paths["cpu_runner"], "-input=2_3_5,2_3_5", "--output", "2_3_5", f"--data={fa}", "--data", fb,
             f"--out-data={out}", os.path.join(paths["models"], "add_cpu.so")])
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, np.float32), (a + b).reshape(-1))


def test_cpu_runner_layernorm_and_fmha_models(paths, tmp_path, oracle):
    x = gen_data.gen_data("2_16_96", seed=5, dist="normal")
    g = gen_data.gen_data("96", seed=6, dist="normal", mean=1.0, std=0.02)
    b = gen_data.gen_data("96", seed=7, dist="normal", std=0.02)
    files = [gen_data.save_data(t, str(tmp_path / n)) for t, n in ((x, "x"), (g, "g"), (b, "b"))]
    out = str(tmp_path / "y.dat")
    r = run([paths["cpu_runner"], os.path.join(paths["models"], "layernorm_cpu.so"), "--input",
             "2_16_96,96,96", "--output", "2_16_96", "--data", ",".join(files), "--out-data", out])
    assert r.returncode == 0, r.stderr
    y = np.fromfile(out, np.float32).reshape(2, 16, 96)
    ref = oracle.layernorm(x, g, b)
    assert np.all(np.abs(y - ref) <= 1e-5 * np.abs(ref) + 1e-6)

    qkv = (gen_data.gen_data("2_40_3_2_64", "f32", seed=8, dist="normal") / 8).astype(np.float16)
    fq = gen_data.save_data(qkv, str(tmp_path / "qkv"))
    assert fq.endswith("qkv_float16_2_40_3_2_64.dat")
    out = str(tmp_path / "o.dat")
    r = run([paths["cpu_runner"], os.path.join(paths["models"], "fmha_cpu.so"), "--dtype", "f16", "--input",
             "2_40_3_2_64", "--output", "2_40_128", "--data", fq, "--out-data", out])
    assert r.returncode == 0, r.stderr
    o = np.fromfile(out, np.float16).reshape(2, 40, 128).astype(np.float32)
    assert np.abs(o - oracle.fmha(qkv)).max() <= 2e-3


def test_runner_error_paths_are_reported(paths, tmp_path):
    model = os.path.join(paths["models"], "add_cpu.so")
    # data count != input count
    small = str(tmp_path / "small.dat")
    np.zeros(10, np.float32).tofile(small)
    r = run([paths["cpu_runner"], model, "--data", small])
    assert r.returncode != 0 and "Data num not equal input num!" in r.stderr
    # missing entry point
    r = run([paths["cpu_runner"], model, "--func", "no_such_symbol"])
    assert r.returncode != 0 and "Failed to find run function" in r.stderr
    # missing library
    r = run([paths["cpu_runner"], str(tmp_path / "nope.so")])
    assert r.returncode != 0 and "Failed to open library" in r.stderr
    # unknown flag, missing positional
    r = run([paths["cpu_runner"], model, "--bogus"])
    assert r.returncode == 1 and "Failed to parse options" in r.stderr
    r = run([paths["cpu_runner"]])
    assert r.returncode == 1 and "positional" in r.stderr
    # unknown dtype
    r = run([paths["cpu_runner"], model, "--dtype", "f64"])
    assert r.returncode != 0 and "Not Implemented type!" in r.stderr


def test_short_data_file_reports_wrong_file_size(paths, tmp_path):
    """A file shorter than the tensor prints 'Wrong File size' (the reference
    then runs on a null buffer; the loader's message is what is kept)."""
    small = str(tmp_path / "small.dat")
    np.zeros(10, np.float32).tofile(small)
    # use a 1-element-output model shape so nothing is dereferenced: shapes of 0 rows
    r = run([paths["cpu_runner"], os.path.join(paths["models"], "add_cpu.so"), "--input", "0_4_4,0_4_4",
             "--output", "0_4_4", "--data", f"{small},{small}"])
    assert r.returncode == 0
    big = run([paths["cpu_runner"], os.path.join(paths["models"], "add_cpu.so"), "--input", "0_4_4,1_4_4",
               "--output", "0_4_4", "--data", f"{small},{small}"])
    assert "Wrong File size" in big.stderr


def test_gpu_runner_links_and_prints_help(paths):
    r = run([paths["gpu_runner"], "--help"])
    assert r.returncode == 0
    for flag in ("--func", "--out-data", "--rerun", "--ops", "--input", "--output", "--data", "--dtype"):
        assert flag in r.stdout


def test_lib_generate_cpu_model_from_llvm_ir(paths, pkg, tmp_path, oracle):
    """multi-device-lib-generate (the reference's tool of that name,
    tools/multi-device-lib-generate/multi-device-lib-generate.cpp:41-67): model
    LLVM IR -> opt -> llc -> shared library, temporaries removed unless asked
    for, and the library runs under the CPU runner."""
    import shutil
    tool = os.path.join(pkg.BIN_DIR, "multi-device-lib-generate")
    gen = os.path.join(paths["models"], "generated")
    # the build already took the add model through the tool; that library must run
    a = gen_data.gen_data("2_33_65", seed=5, dist="uniform")
    b = gen_data.gen_data("2_33_65", seed=6, dist="uniform")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    out = str(tmp_path / "c.dat")
    r = run([paths["cpu_runner"], os.path.join(gen, "add_cpu.so"), "--input", "2_33_65,2_33_65", "--output", "2_33_65",
             "--data", f"{fa},{fb}", "--out-data", out])
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, np.float32).view(np.uint32), oracle.add_f32(a, b).reshape(-1).view(np.uint32))
    # a fresh run of the tool on the same IR, in a scratch directory
    ll = str(tmp_path / "model.ll")
    shutil.copy(os.path.join(gen, "add_cpu.ll"), ll)
    r = run([tool, ll, "--saveObject"])
    assert r.returncode == 0, r.stderr
    assert os.path.exists(tmp_path / "model.so") and os.path.exists(tmp_path / "model.o")
    assert not os.path.exists(tmp_path / "model_opt.ll")
    r = run([tool, ll, "-o", str(tmp_path / "named"), "--saveOptIR", "-O3"])
    assert r.returncode == 0, r.stderr
    assert os.path.exists(tmp_path / "named.so") and os.path.exists(tmp_path / "model_opt.ll")
    r = run([paths["cpu_runner"], str(tmp_path / "named.so"), "--input", "2_33_65,2_33_65", "--output", "2_33_65",
             "--data", f"{fa},{fb}", "--out-data", out])
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, np.float32).view(np.uint32), oracle.add_f32(a, b).reshape(-1).view(np.uint32))
    # an invalid -o is ignored with a note, as the reference does (:157-166)
    r = run([tool, ll, "-o", str(tmp_path) + "/.."])
    assert r.returncode == 0 and "Invalid -o option value" in r.stderr


def test_lib_generate_gpu_artifacts_and_errors(pkg, paths, tmp_path):
    """--device gpu also turns the kernel source (AMDGPU LLVM IR or HIP) into
    ops.hsaco beside it; the build's own run of it left a code object holding the
    generated-style kernel.  Failures name the step and return non-zero."""
    tool = os.path.join(pkg.BIN_DIR, "multi-device-lib-generate")
    gen = os.path.join(paths["models"], "generated")
    blob = open(os.path.join(gen, "ops.hsaco"), "rb").read()
    assert blob[:4] == b"\x7fELF" and b"main_graph_kernel" in blob
    assert os.path.exists(os.path.join(gen, "add_gpu.so"))
    r = run([tool, str(tmp_path / "missing.ll")])
    assert r.returncode != 0 and "Failed to open input" in r.stderr
    bad = tmp_path / "bad.ll"
    bad.write_text("this is not LLVM IR\n")
    r = run([tool, str(bad)])
    assert r.returncode != 0 and "Opt LLVM IR wrong." in r.stderr and "Command execution failed." in r.stderr
    r = run([tool, os.path.join(gen, "add_cpu.ll"), "-o", str(tmp_path / "x"), "--device", "tpu"])
    assert r.returncode != 0 and "--device is cpu or gpu" in r.stderr
    r = run([tool, os.path.join(gen, "add_gpu.ll"), "-o", str(tmp_path / "y"), "--device", "gpu",
             "--ops", str(tmp_path / "nope.hip")])
    assert r.returncode != 0 and "kernel source not found" in r.stderr


REF_ADD_LL = "/root/reference/examples/add.ll"


@pytest.mark.skipif(not os.path.exists(REF_ADD_LL), reason="the reference tree is not present on this machine")
def test_reference_add_ll_through_lib_generate_and_cpu_runner(pkg, paths, tmp_path, oracle):
    """The reference's one pre-lowered model (examples/add.ll:8-104, entry
    _mlir_ciface_main_graph with outputs first) goes through this build's
    multi-device-lib-generate and runs under this build's CPU runner with the
    reference's own default shapes; the result is bit-exact."""
    import shutil
    ll = str(tmp_path / "add.ll")
    shutil.copy(REF_ADD_LL, ll)
    r = run([os.path.join(pkg.BIN_DIR, "multi-device-lib-generate"), ll, "-o", str(tmp_path / "add")])
    assert r.returncode == 0, r.stderr
    a = gen_data.gen_data("3_640_640", seed=41, dist="uniform")
    b = gen_data.gen_data("3_640_640", seed=42, dist="uniform")
    fa, fb = gen_data.save_data(a, str(tmp_path / "a")), gen_data.save_data(b, str(tmp_path / "b"))
    out = str(tmp_path / "c.dat")
    r = run([paths["cpu_runner"], str(tmp_path / "add.so"), "--data", f"{fa},{fb}", "--out-data", out, "--rerun", "2"])
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(out, np.float32).view(np.uint32), oracle.add_f32(a, b).reshape(-1).view(np.uint32))
