"""ctypes bindings of the MI355X device runtime and kernel library.

The product is the pair of C-ABI shared libraries built from ``csrc/``
(``lib/libmgpu_hip_runtime.so``: the ``mgpu*`` stream/event/buffer/launch
wrappers, ``lib/libmgpu_hip_ops.so``: LayerNorm, fused attention, add, casts,
GEMM epilogues and the transformer layers).  This module only loads them and
marshals arguments: device memory and streams come from the caller (PyTorch
tensors in the tests and the bench), every computation happens inside the HIP
libraries.  There is no fallback: a missing library or a failing call raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
BIN_DIR = os.path.join(_HERE, "bin")
RUNTIME_LIB = os.path.join(LIB_DIR, "libmgpu_hip_runtime.so")
OPS_LIB = os.path.join(LIB_DIR, "libmgpu_hip_ops.so")
OPS_MODULE = os.path.join(LIB_DIR, "ops.hsaco")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")


class MgpuError(RuntimeError):
    """A kernel-library entry point reported a failure."""


def build(force: bool = True, jobs: int = 8) -> None:
    """Compile every HIP / C++ target in-tree with the package Makefile."""
    cmd = ["make", "-C", _HERE, f"-j{jobs}", "all"]
    if force:
        cmd.insert(1, "-B")
    subprocess.check_call(cmd)


def is_built() -> bool:
    return os.path.exists(RUNTIME_LIB) and os.path.exists(OPS_LIB)


_c_void_p, _c_int32, _c_int64, _c_float, _c_size_t = (
    ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/mgpu_ops.h
OPS_SIGNATURES = {
    "mgpuOpsInit": (None, []),
    "mgpuOpsDeinit": (None, []),
    "mgpuOpsTakeLastError": (ctypes.c_char_p, []),
    "mgpuLLMOpsCacheWeights": (None, [_c_int32]),
    "mgpuAddF32": (None, [_c_void_p] * 3 + [_c_int64, _c_void_p]),
    "mgpuLayerNormF32": (None, [_c_void_p] * 4 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuLayerNormF16": (None, [_c_void_p] * 4 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuLayerNormBF16": (None, [_c_void_p] * 4 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuCastLayerNormF32ToF16": (None, [_c_void_p] * 5 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuAddResidualPreLayerNormF32": (None, [_c_void_p] * 6 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuAddResidualPreLayerNormF16": (None, [_c_void_p] * 6 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuAddResidualPreLayerNormBF16": (None, [_c_void_p] * 6 + [_c_float, _c_int32, _c_int32, _c_void_p]),
    "mgpuFusedMHAF16": (None, [_c_void_p] * 3 + [_c_int32] * 4 + [_c_float, _c_int32, _c_void_p]),
    "mgpuFusedMHABF16": (None, [_c_void_p] * 3 + [_c_int32] * 4 + [_c_float, _c_int32, _c_void_p]),
    "mgpuFusedMHAF16CuSeqlens": (None, [_c_void_p] * 3 + [_c_int32] * 4 + [_c_float, _c_int32, _c_void_p]),
    "mgpuFusedMHABF16CuSeqlens": (None, [_c_void_p] * 3 + [_c_int32] * 4 + [_c_float, _c_int32, _c_void_p]),
    "mgpuCastF32ToF16": (None, [_c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "mgpuCastF16ToF32": (None, [_c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "mgpuCastF32ToBF16": (None, [_c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "mgpuCastBF16ToF32": (None, [_c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "mgpuAddFusedQKVBiasTransposeF16": (None, [_c_void_p] * 5 + [_c_int32] * 5 + [_c_void_p]),
    "mgpuAddFusedQKVBiasTransposeBF16": (None, [_c_void_p] * 5 + [_c_int32] * 5 + [_c_void_p]),
    "mgpuMatmul": (None, [_c_void_p] * 4 + [_c_int64] * 3 + [_c_void_p]),
    "mgpuConv2d": (None, [_c_void_p] * 5 + [_c_int64] * 17 + [ctypes.c_bool] * 2 + [_c_void_p]),
    "mgpuPool2d": (None, [_c_void_p] * 2 + [_c_int64] * 15 + [_c_void_p]),
    "mgpuMatmulExF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuMatmulExBF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuPackWeight16": (None, [_c_void_p] * 2 + [_c_int64] * 2 + [_c_void_p]),
    "mgpuMatmulExPackedF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuMatmulExPackedBF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuGemmMfmaF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuGemmMfmaBF16": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuMatmulExF32": (None, [_c_void_p] * 5 + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p]),
    "mgpuLLMDecodingContextLayer": (None, [_c_void_p] * 9 + [_c_int64] * 5 + [ctypes.c_bool] * 3 + [_c_void_p]),
    "mgpuBertEncoderLayerF16": (None, [_c_void_p] * 15 + [_c_int64] * 5 + [_c_float, _c_void_p]),
    "mgpuBertEncoderLayerF16NoAlloc": (None, [_c_void_p] * 15 + [_c_int64] * 5 + [_c_float, _c_void_p]),
}

# mirrors include/mgpu_runtime.h
RUNTIME_SIGNATURES = {
    "mgpuModuleFileLoad": (None, [ctypes.c_char_p]),
    "mgpuModuleUnload": (None, []),
    "mgpuModuleGetFunction": (_c_void_p, [ctypes.c_char_p]),
    "mgpuLaunchKernel": (None, [_c_void_p] + [ctypes.c_ssize_t] * 6 + [_c_int32, _c_void_p,
                                ctypes.POINTER(_c_void_p), ctypes.POINTER(_c_void_p)]),
    "mgpuStreamCreate": (_c_void_p, []),
    "mgpuStreamDestroy": (None, [_c_void_p]),
    "mgpuStreamSynchronize": (None, [_c_void_p]),
    "mgpuStreamWaitEvent": (None, [_c_void_p, _c_void_p]),
    "mgpuEventCreate": (_c_void_p, []),
    "mgpuEventCreateWithStream": (_c_void_p, [_c_void_p]),
    "mgpuEventEnableTimeCreate": (_c_void_p, []),
    "mgpuEventDestroy": (None, [_c_void_p]),
    "mgpuEventSynchronize": (None, [_c_void_p]),
    "mgpuEventRecord": (None, [_c_void_p, _c_void_p]),
    "mgpuEventElapsedTime": (_c_float, [_c_void_p, _c_void_p]),
    "mgpuMemAlloc": (_c_void_p, [ctypes.c_uint64, _c_void_p]),
    "mgpuMemFree": (None, [_c_void_p, _c_void_p]),
    "mgpuMemAllocAsync": (_c_void_p, [ctypes.c_uint64, _c_void_p]),
    "mgpuMemFreeAsync": (None, [_c_void_p, _c_void_p]),
    "mgpuMemcpy": (None, [_c_void_p, _c_void_p, _c_size_t, _c_void_p]),
    "mgpuMemset32": (None, [_c_void_p, ctypes.c_uint, _c_size_t, _c_void_p]),
    "mgpuMemset16": (None, [_c_void_p, ctypes.c_ushort, _c_size_t, _c_void_p]),
    "mgpuMemHostRegister": (None, [_c_void_p, ctypes.c_uint64]),
    "mgpuMemHostUnregister": (None, [_c_void_p]),
    "mgpuMemHostRegisterMemRef": (None, [_c_int64, _c_void_p, _c_int64]),
    "mgpuMemHostUnregisterMemRef": (None, [_c_int64, _c_void_p, _c_int64]),
    "mgpuSetDefaultDevice": (None, [_c_int32]),
    "mgpuRuntimeTakeLastError": (_c_int32, []),
}


def _load(path: str, signatures) -> ctypes.CDLL:
    if not os.path.exists(path):
        raise MgpuError(f"{path} is not built; run `make -C {_HERE}` (or __graft_entry__.build())")
    lib = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    for name, (restype, argtypes) in signatures.items():
        fn = getattr(lib, name)  # AttributeError if the export is missing: fail loudly
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


_runtime = None
_ops = None
_ops_initialised = False


def runtime() -> ctypes.CDLL:
    global _runtime
    if _runtime is None:
        _runtime = _load(RUNTIME_LIB, RUNTIME_SIGNATURES)
    return _runtime


BENCH_LIB = os.path.join(LIB_DIR, "libmgpu_bench_loops.so")
_bench = None


def bench_loops() -> ctypes.CDLL:
    """The benchmark's launch loops, ceiling probes, attention profile entry and GEMM tuner
    (measurement plumbing, not part of the kernel library)."""
    global _bench
    if _bench is None:
        if not os.path.exists(BENCH_LIB):
            raise MgpuError(f"{BENCH_LIB} is not built")
        ops(init=False)  # the loops call into the kernel library
        lib = ctypes.CDLL(BENCH_LIB)
        f32 = ctypes.c_float
        for name in ("mgpuBenchLayerNormF32", "mgpuBenchLayerNormF16", "mgpuBenchAddF32", "mgpuBenchFusedMHAF16",
                     "mgpuBenchBertEncoderLayerF16", "mgpuProbeCopy", "mgpuProbeCombine", "mgpuProbeMfma",
                     "mgpuProbeFmhaLoop", "mgpuProbeLdsRead"):
            getattr(lib, name).restype = f32
        lib.mgpuBenchFusedMHAF16Profile.restype = _c_int64
        lib.mgpuBenchFusedMHAF16Profile.argtypes = [_c_void_p, _c_void_p] + [_c_int32] * 3 + [_c_float, _c_void_p,
                                                                                               _c_void_p]
        lib.mgpuBenchTuneMatmulEx.restype = _c_int32
        lib.mgpuBenchTuneMatmulEx.argtypes = [_c_int32] + [_c_int64] * 3 + [_c_int32] * 3 + [_c_void_p] * 3
        _bench = lib
    return _bench


def ops(init: bool = True) -> ctypes.CDLL:
    """The kernel library; ``init`` also runs mgpuOpsInit() once (needs a GPU)."""
    global _ops, _ops_initialised
    if _ops is None:
        _ops = _load(OPS_LIB, OPS_SIGNATURES)
    if init and not _ops_initialised:
        _ops.mgpuOpsInit()
        _check(_ops)
        _ops_initialised = True
    return _ops


def _check(lib) -> None:
    msg = lib.mgpuOpsTakeLastError()
    if msg is not None:
        raise MgpuError(msg.decode())


# --------------------------------------------------------------------------
# Tensor-level helpers (torch tensors on the GPU; torch only supplies memory
# and the stream handle).
# --------------------------------------------------------------------------

def _stream_handle(stream=None) -> int:
    import torch
    s = stream if stream is not None else torch.cuda.current_stream()
    return s.cuda_stream


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise MgpuError("expected a tensor in device memory")
    if not t.is_contiguous():
        raise MgpuError("expected a contiguous tensor")
    return t.data_ptr()


def _suffix(dtype) -> str:
    import torch
    return {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16"}[dtype]


def add(a, b, out=None, stream=None):
    import torch
    assert a.dtype == torch.float32 and b.dtype == torch.float32 and a.shape == b.shape
    if out is None:
        out = torch.empty_like(a)
    lib = ops()
    lib.mgpuAddF32(_ptr(a), _ptr(b), _ptr(out), a.numel(), _stream_handle(stream))
    _check(lib)
    return out


def layer_norm(x, gamma, beta, eps: float = 1e-5, out=None, stream=None):
    import torch
    n = x.shape[-1]
    m = x.numel() // n if n else 0
    if out is None:
        out = torch.empty_like(x)
    lib = ops()
    getattr(lib, "mgpuLayerNorm" + _suffix(x.dtype))(
        _ptr(x), _ptr(gamma), _ptr(beta), _ptr(out), eps, m, n, _stream_handle(stream))
    _check(lib)
    return out


def cast_layer_norm(x, gamma, beta, eps: float = 1e-5, stream=None):
    """fp32 x -> (fp16 copy of x, LayerNorm of that copy in fp16), one pass."""
    import torch
    assert x.dtype == torch.float32
    n = x.shape[-1]
    m = x.numel() // n if n else 0
    cast = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    normed = torch.empty_like(cast)
    lib = ops()
    lib.mgpuCastLayerNormF32ToF16(_ptr(x), _ptr(gamma), _ptr(beta), _ptr(cast), _ptr(normed), eps, m, n,
                                  _stream_handle(stream))
    _check(lib)
    return cast, normed


def add_residual_layer_norm(x, residual, gamma, beta, eps: float = 1e-5, stream=None):
    import torch
    n = x.shape[-1]
    m = x.numel() // n if n else 0
    summed = torch.empty_like(x)
    normed = torch.empty_like(x)
    lib = ops()
    getattr(lib, "mgpuAddResidualPreLayerNorm" + _suffix(x.dtype))(
        _ptr(x), _ptr(residual), _ptr(gamma), _ptr(beta), _ptr(summed), _ptr(normed), eps, m, n,
        _stream_handle(stream))
    _check(lib)
    return summed, normed


def fused_mha(qkv, seqlens=None, scale=None, causal: bool = False, out=None, stream=None):
    """qkv [B,S,3,H,D] fp16/bf16 -> [B,S,H*D]."""
    import torch
    B, S, three, H, D = qkv.shape
    assert three == 3
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    if out is None:
        out = torch.empty((B, S, H * D), dtype=qkv.dtype, device=qkv.device)
    if seqlens is not None:
        assert seqlens.dtype == torch.int32 and seqlens.numel() == B
    lib = ops()
    getattr(lib, "mgpuFusedMHA" + _suffix(qkv.dtype))(
        _ptr(qkv), _ptr(seqlens), _ptr(out), B, S, H, D, scale, 1 if causal else 0,
        _stream_handle(stream))
    _check(lib)
    return out


def fused_mha_cu_seqlens(qkv, cu_seqlens, max_s: int, scale=None, causal: bool = False, out=None, stream=None):
    """qkv [total,3,H,D] fp16/bf16 packed back to back, cu_seqlens int32 [B+1] -> [total,H*D]."""
    import torch
    total, three, H, D = qkv.shape
    assert three == 3 and cu_seqlens.dtype == torch.int32
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    if out is None:
        out = torch.empty((total, H * D), dtype=qkv.dtype, device=qkv.device)
    lib = ops()
    getattr(lib, "mgpuFusedMHA" + _suffix(qkv.dtype) + "CuSeqlens")(
        _ptr(qkv), _ptr(cu_seqlens), _ptr(out), cu_seqlens.numel() - 1, max_s, H, D, scale, 1 if causal else 0,
        _stream_handle(stream))
    _check(lib)
    return out


def cast_f32_to_f16(x, stream=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    lib = ops()
    lib.mgpuCastF32ToF16(_ptr(out), _ptr(x), x.numel(), _stream_handle(stream))
    _check(lib)
    return out


def cast_f16_to_f32(x, stream=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    lib = ops()
    lib.mgpuCastF16ToF32(_ptr(out), _ptr(x), x.numel(), _stream_handle(stream))
    _check(lib)
    return out


def cast_f32_to_bf16(x, stream=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    lib = ops()
    lib.mgpuCastF32ToBF16(_ptr(out), _ptr(x), x.numel(), _stream_handle(stream))
    _check(lib)
    return out


def cast_bf16_to_f32(x, stream=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    lib = ops()
    lib.mgpuCastBF16ToF32(_ptr(out), _ptr(x), x.numel(), _stream_handle(stream))
    _check(lib)
    return out


def qkv_bias_transpose(qkv, bias, stream=None):
    """qkv [B,S,3,H,D] fp16 or bf16 (updated in place with the bias) -> q, k, v [B,H,S,D]."""
    import torch
    B, S, _, H, D = qkv.shape
    q = torch.empty((B, H, S, D), dtype=qkv.dtype, device=qkv.device)
    k = torch.empty_like(q)
    v = torch.empty_like(q)
    lib = ops()
    fn = lib.mgpuAddFusedQKVBiasTransposeBF16 if qkv.dtype == torch.bfloat16 else lib.mgpuAddFusedQKVBiasTransposeF16
    fn(_ptr(q), _ptr(k), _ptr(v), _ptr(qkv), _ptr(bias), B, S, B * S, H, D, _stream_handle(stream))
    _check(lib)
    return q, k, v


ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2


def pack_weight(w, stream=None):
    """mgpuPackWeight16: the K-major copy ([N, K]) of a 16-bit [K, N] weight, for matmul_ex(kernel="packed")."""
    import torch
    assert w.dtype in (torch.float16, torch.bfloat16) and w.dim() == 2 and w.is_contiguous()
    K, N = w.shape
    packed = torch.empty((N, K), dtype=w.dtype, device=w.device)
    lib = ops()
    lib.mgpuPackWeight16(_ptr(packed), _ptr(w), K, N, _stream_handle(stream))
    _check(lib)
    return packed


def matmul_ex(x, w, bias=None, residual=None, act: int = ACT_NONE, stream=None, kernel: str = "auto"):
    """kernel "auto": mgpuMatmulEx*, i.e. the library or the hand-written MFMA kernel as
    the committed table and the fixed rule of the library say; "mfma": the hand-written kernel itself (fp16 / bf16, M a multiple
    of 128, N of 128 or 96, K of 32); "packed": mgpuMatmulExPacked*, w being the [N, K] copy pack_weight made."""
    import torch
    M, K = x.shape
    if kernel == "packed":
        N, K2 = w.shape
    else:
        K2, N = w.shape
    assert K == K2
    out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    lib = ops()
    if kernel == "mfma":
        fn = {torch.float16: lib.mgpuGemmMfmaF16, torch.bfloat16: lib.mgpuGemmMfmaBF16}[x.dtype]
    elif kernel == "packed":
        fn = {torch.float16: lib.mgpuMatmulExPackedF16, torch.bfloat16: lib.mgpuMatmulExPackedBF16}[x.dtype]
    else:
        assert kernel == "auto", kernel
        fn = {torch.float16: lib.mgpuMatmulExF16, torch.bfloat16: lib.mgpuMatmulExBF16,
              torch.float32: lib.mgpuMatmulExF32}[x.dtype]
    fn(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), _ptr(residual), M, N, K,
       1 if bias is not None else 0, act, 1 if residual is not None else 0, _stream_handle(stream))
    _check(lib)
    return out


def _conv_out(size, k, pl, pr, s, d=1):
    return (size + pl + pr - d * (k - 1) - 1) // s + 1


def conv2d(x, w, bias, post_add=None, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), relu=False, stream=None):
    """NCHW fp32; pad = (top, left, bottom, right)."""
    import torch
    N, IC, H, W = x.shape
    OC, IC2, KH, KW = w.shape
    assert IC == IC2
    OH = _conv_out(H, KH, pad[0], pad[2], stride[0], dilation[0])
    OW = _conv_out(W, KW, pad[1], pad[3], stride[1], dilation[1])
    out = torch.empty((N, OC, OH, OW), dtype=x.dtype, device=x.device)
    lib = ops()
    lib.mgpuConv2d(_ptr(x), _ptr(w), _ptr(bias), _ptr(out), _ptr(post_add), N, IC, H, W, OC, KH, KW, OH, OW,
                   pad[0], pad[1], pad[2], pad[3], stride[0], stride[1], dilation[0], dilation[1],
                   post_add is not None, relu, _stream_handle(stream))
    _check(lib)
    return out


def pool2d(x, kernel, pad=(0, 0, 0, 0), stride=(1, 1), method="max", stream=None):
    """NCHW fp32; method "max" or "avg" (average counts the padding)."""
    import torch
    N, C, H, W = x.shape
    OH = _conv_out(H, kernel[0], pad[0], pad[2], stride[0])
    OW = _conv_out(W, kernel[1], pad[1], pad[3], stride[1])
    out = torch.empty((N, C, OH, OW), dtype=x.dtype, device=x.device)
    lib = ops()
    lib.mgpuPool2d(_ptr(x), _ptr(out), N, C, H, W, OH, OW, kernel[0], kernel[1], pad[0], pad[1], pad[2], pad[3],
                   stride[0], stride[1], 0 if method == "max" else 1, _stream_handle(stream))
    _check(lib)
    return out


def decoding_context_layer(x, wqkv, wo, bo, w1, b1, w2, b2, heads: int, causal: bool = True,
                           relu: bool = True, norm_first: bool = True, stream=None):
    import torch
    B, S, d = x.shape
    ffn = w1.shape[1]
    out = torch.empty_like(x)
    lib = ops()
    lib.mgpuLLMDecodingContextLayer(_ptr(x), _ptr(wqkv), _ptr(wo), _ptr(bo), _ptr(w1), _ptr(b1),
                                    _ptr(w2), _ptr(b2), _ptr(out), B, S, d, ffn, heads, norm_first,
                                    causal, relu, _stream_handle(stream))
    _check(lib)
    return out


def bert_encoder_layer(x, wqkv, bqkv, wo, bo, g1, be1, w1, b1, w2, b2, g2, be2, heads: int,
                       seqlens=None, eps: float = 1e-5, out=None, stream=None, no_alloc: bool = False):
    """no_alloc: the entry point whose temporaries live in the library's fixed
    device array (the caller supplies ``out``: nothing is allocated then)."""
    import torch
    B, S, d = x.shape
    ffn = w1.shape[1]
    if out is None:
        out = torch.empty_like(x)
    lib = ops()
    fn = lib.mgpuBertEncoderLayerF16NoAlloc if no_alloc else lib.mgpuBertEncoderLayerF16
    fn(_ptr(x), _ptr(wqkv), _ptr(bqkv), _ptr(wo), _ptr(bo), _ptr(g1),
                                _ptr(be1), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(b2), _ptr(g2),
                                _ptr(be2), _ptr(seqlens), _ptr(out), B, S, d, ffn, heads, eps,
                                _stream_handle(stream))
    _check(lib)
    return out
