"""Argument validation of the kernel library's C ABI: a bad call prints,
records the message for mgpuOpsTakeLastError() and launches nothing - so these
run without a GPU."""
import ctypes

import pytest


@pytest.fixture(scope="module")
def lib(pkg):
    return pkg.ops(init=False)


def take(lib):
    m = lib.mgpuOpsTakeLastError()
    return None if m is None else m.decode()


def test_no_error_initially_and_query_clears(lib):
    take(lib)
    assert take(lib) is None
    lib.mgpuFusedMHAF16(1, None, 1, 1, 1, 1, 264, 0.125, 0, None)
    assert "head_dim must be a multiple of 8 between 8 and 256" in take(lib)
    assert take(lib) is None


def test_fmha_rejects_bad_arguments(lib):
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) // 16 * 16
    lib.mgpuFusedMHAF16(None, None, p16, 1, 1, 1, 64, 0.125, 0, None)
    assert "null pointer" in take(lib)
    lib.mgpuFusedMHAF16(p16 + 2, None, p16, 1, 1, 1, 64, 0.125, 0, None)
    assert "16-byte aligned" in take(lib)
    lib.mgpuFusedMHAF16(p16, None, p16, 1, 1, 1, 64, 0.0, 0, None)
    assert "scale" in take(lib)
    lib.mgpuFusedMHAF16(p16, None, p16, -1, 1, 1, 64, 0.125, 0, None)
    assert "negative" in take(lib)
    # empty problems are accepted and do nothing
    lib.mgpuFusedMHAF16(None, None, None, 0, 128, 12, 64, 0.125, 0, None)
    assert take(lib) is None


def test_layernorm_and_add_reject_bad_arguments(lib):
    lib.mgpuLayerNormF32(None, None, None, None, 1e-5, 4, 8, None)
    assert "null pointer" in take(lib)
    lib.mgpuLayerNormF32(None, None, None, None, 1e-5, -1, 8, None)
    assert "negative" in take(lib)
    lib.mgpuLayerNormF16(None, None, None, None, 1e-5, 0, 8, None)
    assert take(lib) is None
    lib.mgpuAddResidualPreLayerNormF16(1, None, 1, 1, None, 1, 1e-5, 2, 8, None)
    assert "null pointer" in take(lib)
    lib.mgpuAddF32(None, None, None, 5, None)
    assert "null pointer" in take(lib)
    lib.mgpuAddF32(None, None, None, -5, None)
    assert "negative" in take(lib)
    lib.mgpuAddF32(None, None, None, 0, None)
    assert take(lib) is None


def test_matmul_and_layers_reject_bad_arguments(lib):
    # The calls below hand the library made-up pointers and count on it refusing them before
    # any launch because gpuOpsInit() has not run.  Ask that with null pointers first: where
    # another test of this process has initialised the library, the answer is "null pointer"
    # and the made-up pointers stay out of it.
    lib.mgpuMatmulExF16(None, None, None, None, None, 4, 4, 4, 0, 0, 0, None)
    if "gpuOpsInit" not in (take(lib) or ""):
        pytest.skip("the kernel library is already initialised in this process")
    lib.mgpuMatmulExF16(1, 1, None, 1, None, 4, 4, 4, 0, 0, 0, None)
    assert "gpuOpsInit" in take(lib)  # library not initialised in this process
    lib.mgpuMatmulExF16(1, 1, None, 1, None, -4, 4, 4, 0, 0, 0, None)
    assert "negative" in take(lib)
    lib.mgpuLLMDecodingContextLayer(1, 1, 1, 1, 1, 1, 1, 1, 1, 2, 8, 512, 1024, 8, True, True, True, None)
    assert "gpuOpsInit" in take(lib)
    lib.mgpuBertEncoderLayerF16(*([1] * 13), None, 1, 2, 8, 768, 3072, 64, 1e-5, None)
    assert "multiple of 8 between 8 and 256" in take(lib)
    lib.mgpuAddFusedQKVBiasTransposeF16(16, 16, 16, 16, None, 2, 8, 15, 2, 64, None)
    assert "token_num" in take(lib)
