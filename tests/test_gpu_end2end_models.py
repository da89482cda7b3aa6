"""The reference's End2End test models (test/End2End/GPU/*.mlir) with their own
constants, lowered from device plans and run by multi-device-gpu-runner."""
import os

import numpy as np
import pytest

from test_end2end_models import run_model

pytestmark = pytest.mark.gpu


def gpu_runner(pkg):
    return os.path.join(pkg.BIN_DIR, "multi-device-gpu-runner")


@pytest.mark.parametrize("name", ["add", "add_constant", "add_constant_splat"])
def test_end2end_add_models(pkg, gpu, name, tmp_path, oracle, rng):
    got, ref = run_model(gpu_runner(pkg), name, "gpu", tmp_path, oracle, rng, ("--ops", pkg.OPS_MODULE))
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_end2end_linear(pkg, gpu, tmp_path, oracle, rng):
    """MatMul + Add + Relu as one GEMM call with the ReLU epilogue; true fp32
    products and accumulation (see test_matmul_f32)."""
    got, ref = run_model(gpu_runner(pkg), "linear", "gpu", tmp_path, oracle, rng, ("--ops", pkg.OPS_MODULE))
    assert np.all(np.abs(got - ref) <= 1e-5 * (1.0 + np.abs(ref)))


def test_end2end_conv_and_pool(pkg, gpu, tmp_path, oracle, rng):
    got, ref = run_model(gpu_runner(pkg), "conv", "gpu", tmp_path / "conv", oracle, rng, ("--ops", pkg.OPS_MODULE))
    assert np.all(np.abs(got - ref) <= 1e-4 * (1.0 + np.abs(ref)))
    got, ref = run_model(gpu_runner(pkg), "pool", "gpu", tmp_path / "pool", oracle, rng, ("--ops", pkg.OPS_MODULE))
    assert np.array_equal(got, ref)
