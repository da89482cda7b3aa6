"""The C-ABI libraries load and export every symbol the headers declare (no
compute calls: runs without a GPU)."""
import ctypes
import os
import re
import subprocess

import pytest

from conftest import ROOT

INCLUDE = os.path.join(ROOT, "include")


def _declared(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mgpu[A-Za-z0-9]+)\s*\(", text)))


def _exported(path):
    out = subprocess.check_output(["nm", "-D", "--defined-only", path], text=True)
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_runtime_exports_every_declared_symbol(pkg):
    declared = _declared("mgpu_runtime.h")
    assert len(declared) >= 28
    exported = _exported(pkg.RUNTIME_LIB)
    assert not [s for s in declared if s not in exported]
    assert set(declared) == set(pkg.RUNTIME_SIGNATURES)  # the bindings cover the header exactly


def test_ops_exports_every_declared_symbol(pkg):
    declared = _declared("mgpu_ops.h")
    assert len(declared) >= 20
    exported = _exported(pkg.OPS_LIB)
    assert not [s for s in declared if s not in exported]
    assert set(declared) == set(pkg.OPS_SIGNATURES)


def test_reference_cxx_names_are_exported(pkg):
    """The C++-linkage names of the reference's Kernels/GPU/Ops.h that compiled
    models and the runner link against (Itanium-mangled, hipStream_t)."""
    exported = _exported(pkg.OPS_LIB)
    for sym in ["_Z10gpuOpsInitv", "_Z12gpuOpsDeinitv", "_Z13gpuLLMOpsInitv", "_Z15gpuLLMOpsDeinitv"]:
        assert sym in exported
    demangled = subprocess.check_output(["nm", "-D", "-C", "--defined-only", pkg.OPS_LIB], text=True)
    for name in ["void mgpuLayerNorm<__half>", "void mgpuAddResidualPreLayerNorm<__half>",
                 "void mgpuMatmulEx<__half>", "void mgpuMatmulEx<float>",
                 "void mgpuAddFusedQKVBiasTranspose<__half>", "void invokeCast<__half, float>",
                 "void invokeCast<float, __half>", "void mgpuFusedMHA<__half>"]:
        assert name in demangled, name


def test_libraries_load_without_gpu(pkg):
    pkg.runtime()
    lib = pkg.ops(init=False)
    assert lib.mgpuOpsTakeLastError() is None


def test_headers_compile_as_c():
    """include/*.h are plain C (no HIP or C++ types in the signatures)."""
    src = '#include "mgpu_runtime.h"\n#include "mgpu_ops.h"\nint main(void){return 0;}\n'
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", INCLUDE, "-x", "c", "-"],
                   input=src, text=True, check=True)


def test_code_object_is_built(pkg):
    assert os.path.getsize(pkg.OPS_MODULE) > 0
