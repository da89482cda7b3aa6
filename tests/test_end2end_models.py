"""The reference's End2End test models (test/End2End/CPU/*.mlir: add, add with
a tensor constant, add with a splat constant, linear, conv, pool) through the
plan lowering and multi-device-cpu-runner, with the constants those files
embed.  The reference's lit RUN lines only check that its pipeline exits 0;
here the models run and the results are compared with the oracle.  No GPU."""
import os
import subprocess

import numpy as np
import pytest

import end2end_models as e2e
from conftest import ROOT

CPU_RUNNER = os.path.join(ROOT, "multi-device-model-compiler_amd", "bin", "multi-device-cpu-runner")


def run_model(runner, name, device, tmp_path, oracle, rng, extra=()):
    plan, in_shapes, out_shape, ref = e2e.build(name, str(tmp_path), device)
    inputs, files = [], []
    for i, s in enumerate(in_shapes):
        a = rng.uniform(-1, 1, s).astype(np.float32)
        f = str(tmp_path / f"in{i}.dat")
        a.tofile(f)
        inputs.append(a)
        files.append(f)
    out = str(tmp_path / "out.dat")
    r = subprocess.run([runner, plan, "--data", ",".join(files), "--out-data", out, *extra],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "failed with" not in r.stderr, r.stderr
    return np.fromfile(out, np.float32).reshape(out_shape), ref(oracle, *inputs)


def test_fixture_constants_are_the_reference_files_constants():
    c = e2e.CONSTANTS
    assert c["add_constant"].shape == (2, 10, 10) and c["add_constant_splat"].shape == (2, 10, 10)
    assert np.all(c["add_constant_splat"] == 1.0)
    # first values as printed in test/End2End/GPU/*.mlir (hex 0x2A4DBB3E, list head -0.04741868, hex 0x8B2F90BB)
    assert c["add_constant"].reshape(-1)[0] == np.frombuffer(bytes.fromhex("2A4DBB3E"), "<f4")[0]
    assert c["linear_bias"][0] == np.float32(-0.04741868)
    assert c["linear_weight"].reshape(-1)[0] == np.frombuffer(bytes.fromhex("F9D20CBE"), "<f4")[0]
    assert c["conv_weight"].reshape(-1)[0] == np.frombuffer(bytes.fromhex("8B2F90BB"), "<f4")[0]
    assert c["conv_bias"][0] == np.float32(-0.0532348156)
    assert e2e.MODELS["conv"]["pad"] == [1, 1, 1, 1] and e2e.MODELS["pool"]["kernel"] == [4, 4]


@pytest.mark.parametrize("name", ["add", "add_constant", "add_constant_splat"])
def test_end2end_add_models_on_the_cpu_runner(name, tmp_path, oracle, rng):
    got, ref = run_model(CPU_RUNNER, name, "cpu", tmp_path, oracle, rng)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_end2end_linear_on_the_cpu_runner(tmp_path, oracle, rng):
    got, ref = run_model(CPU_RUNNER, "linear", "cpu", tmp_path, oracle, rng)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)


def test_end2end_pool_on_the_cpu_runner(tmp_path, oracle, rng):
    got, ref = run_model(CPU_RUNNER, "pool", "cpu", tmp_path, oracle, rng)
    assert np.array_equal(got, ref)


def test_end2end_conv_on_the_cpu_runner(tmp_path, oracle, rng):
    got, ref = run_model(CPU_RUNNER, "conv", "cpu", tmp_path, oracle, rng)
    assert np.abs(got - ref).max() <= 1e-4
