"""ctypes front end of the CPU oracle (``oracle.c``): TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the product library never does.  Every
function takes and returns numpy arrays; 16-bit floats travel as ``uint16``
views (``kind`` 1 = fp16, 2 = bf16, 0 = fp32).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_ADD_PATH = os.path.join(_HERE, "_ref", "libadd_ref.so")

KIND_F32, KIND_F16, KIND_BF16 = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile oracle.c (and oracle/_ref when the reference checkout is there)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {a.dtype}")
    return a


def kind_of(a: np.ndarray, bf16: bool = False) -> int:
    if a.dtype == np.float32:
        return KIND_F32
    if a.dtype == np.float16:
        return KIND_F16
    if a.dtype == np.uint16:
        return KIND_BF16 if bf16 else KIND_F16
    raise TypeError(f"unsupported dtype {a.dtype}")


def _bits(a):
    """fp16 arrays are handed over as their uint16 bit patterns."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    return a.view(np.uint16) if a.dtype == np.float16 else a


def num_threads() -> int:
    return lib().oracle_num_threads()


def set_num_threads(n: int) -> None:
    lib().oracle_set_num_threads(ctypes.c_int(n))


def add_f32(a, b, mt: bool = False):
    a, b = _c(a, np.float32), _c(b, np.float32)
    assert a.shape == b.shape
    c = np.empty_like(a)
    fn = lib().oracle_add_f32_mt if mt else lib().oracle_add_f32
    fn(_p(a), _p(b), _p(c), ctypes.c_int64(a.size))
    return c


def layernorm(x, gamma, beta, eps: float = 1e-5, bf16: bool = False):
    kind = kind_of(x, bf16)
    x, gamma, beta = _bits(x), _bits(gamma), _bits(beta)
    n = x.shape[-1]
    m = x.size // n if n else 0
    y = np.empty(x.shape, np.float32)
    lib().oracle_layernorm(_p(x), _p(gamma), _p(beta), _p(y), ctypes.c_double(eps),
                           ctypes.c_int64(m), ctypes.c_int64(n), ctypes.c_int(kind))
    return y


def add_residual_layernorm(x, residual, gamma, beta, eps: float = 1e-5, bf16: bool = False):
    kind = kind_of(x, bf16)
    x, residual, gamma, beta = _bits(x), _bits(residual), _bits(gamma), _bits(beta)
    n = x.shape[-1]
    m = x.size // n if n else 0
    s = np.empty(x.shape, np.float32)
    y = np.empty(x.shape, np.float32)
    lib().oracle_add_residual_layernorm(_p(x), _p(residual), _p(gamma), _p(beta), _p(s), _p(y),
                                        ctypes.c_double(eps), ctypes.c_int64(m),
                                        ctypes.c_int64(n), ctypes.c_int(kind))
    return s, y


def fmha(qkv, seqlens=None, scale=None, causal: bool = False, bf16: bool = False):
    """qkv [B,S,3,H,D] -> out [B,S,H*D] fp32."""
    kind = kind_of(qkv, bf16)
    B, S, three, H, D = qkv.shape
    assert three == 3
    qkv = _bits(qkv)
    if seqlens is not None:
        seqlens = _c(np.asarray(seqlens, np.int32))
        assert seqlens.shape == (B,)
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    out = np.empty((B, S, H * D), np.float32)
    lib().oracle_fmha(_p(qkv), _p(seqlens), _p(out), ctypes.c_int64(B), ctypes.c_int64(S),
                      ctypes.c_int64(H), ctypes.c_int64(D), ctypes.c_double(scale),
                      ctypes.c_int(1 if causal else 0), ctypes.c_int(kind))
    return out


ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2


def gemm(x, w, bias=None, residual=None, act: int = ACT_NONE, bf16: bool = False):
    kind = kind_of(x, bf16)
    M, K = x.shape
    K2, N = w.shape
    assert K == K2
    x, w, bias, residual = _bits(x), _bits(w), _bits(bias), _bits(residual)
    out = np.empty((M, N), np.float32)
    lib().oracle_gemm(_p(x), _p(w), _p(bias), _p(residual), _p(out), ctypes.c_int64(M),
                      ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int(act), ctypes.c_int(kind))
    return out


def cast_f32_to_f16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_cast_f32_to_f16(_p(x), _p(out), ctypes.c_int64(x.size))
    return out.view(np.float16)


def half_to_float(x):
    x = _bits(x)
    out = np.empty(x.shape, np.float32)
    lib().oracle_half_to_float(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def double_to_half(x):
    x = _c(x, np.float64)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_double_to_half(_p(x), _p(out), ctypes.c_int64(x.size))
    return out.view(np.float16)


def float_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_float_to_bf16(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def bf16_to_float(x):
    x = _c(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib().oracle_bf16_to_float(_p(x), _p(out), ctypes.c_int64(x.size))
    return out


def qkv_bias_transpose(qkv, bias, bf16: bool = False):
    kind = kind_of(qkv, bf16)
    B, S, three, H, D = qkv.shape
    qkv, bias = _bits(qkv), _bits(bias)
    q = np.empty((B, H, S, D), np.float32)
    k = np.empty_like(q)
    v = np.empty_like(q)
    lib().oracle_qkv_bias_transpose(_p(qkv), _p(bias), _p(q), _p(k), _p(v), ctypes.c_int64(B),
                                    ctypes.c_int64(S), ctypes.c_int64(H), ctypes.c_int64(D),
                                    ctypes.c_int(kind))
    return q, k, v


def decoding_context_layer(x, wqkv, wo, bo, w1, b1, w2, b2, heads: int, causal: bool = True,
                           act: int = ACT_RELU, norm_first: bool = True):
    """All fp32 in, fp32 out: the signature of mgpuLLMDecodingContextLayer."""
    arrs = [_c(a, np.float32) for a in (x, wqkv, wo, bo, w1, b1, w2, b2)]
    B, S, d = x.shape
    ffn = w1.shape[1]
    out = np.empty((B, S, d), np.float32)
    lib().oracle_decoding_context_layer(*[_p(a) for a in arrs], _p(out), ctypes.c_int64(B),
                                        ctypes.c_int64(S), ctypes.c_int64(d), ctypes.c_int64(ffn),
                                        ctypes.c_int64(heads), ctypes.c_int(1 if norm_first else 0),
                                        ctypes.c_int(1 if causal else 0), ctypes.c_int(act))
    return out


def bert_layer_f16(x, wqkv, bqkv, wo, bo, g1, be1, w1, b1, w2, b2, g2, be2, heads: int,
                   seqlens=None, eps: float = 1e-5):
    arrs = [_bits(_c(a, np.float16)) for a in (x, wqkv, bqkv, wo, bo, g1, be1, w1, b1, w2, b2, g2, be2)]
    B, S, d = x.shape
    ffn = w1.shape[1]
    if seqlens is not None:
        seqlens = _c(np.asarray(seqlens, np.int32))
    out = np.empty((B, S, d), np.float32)
    lib().oracle_bert_layer_f16(*[_p(a) for a in arrs], _p(seqlens), _p(out), ctypes.c_int64(B),
                                ctypes.c_int64(S), ctypes.c_int64(d), ctypes.c_int64(ffn),
                                ctypes.c_int64(heads), ctypes.c_double(eps))
    return out


# --------------------------------------------------------------------------
# oracle/_ref: the reference's own compiled add model (examples/add.ll)
# --------------------------------------------------------------------------

class _MemRef3(ctypes.Structure):
    """MLIR rank-3 memref descriptor, the layout examples/add.ll:80-104 unpacks."""
    _fields_ = [("allocated", ctypes.c_void_p), ("aligned", ctypes.c_void_p),
                ("offset", ctypes.c_int64), ("sizes", ctypes.c_int64 * 3),
                ("strides", ctypes.c_int64 * 3)]


def ref_add_available() -> bool:
    return os.path.exists(_REF_ADD_PATH)


def ref_add_3x640x640(a, b):
    """Run the reference's compiled add model on two (3,640,640) fp32 arrays."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    assert a.shape == (3, 640, 640) and b.shape == (3, 640, 640)
    ref = ctypes.CDLL(_REF_ADD_PATH)
    libc = ctypes.CDLL(None)
    libc.free.argtypes = [ctypes.c_void_p]

    def desc(arr):
        d = _MemRef3()
        d.allocated = d.aligned = arr.ctypes.data
        d.offset = 0
        d.sizes[:] = [3, 640, 640]
        d.strides[:] = [409600, 640, 1]
        return d

    da, db, out = desc(a), desc(b), _MemRef3()
    ref._mlir_ciface_main_graph(ctypes.byref(out), ctypes.byref(da), ctypes.byref(db))
    res = np.ctypeslib.as_array(ctypes.cast(out.aligned, ctypes.POINTER(ctypes.c_float)),
                                shape=(3, 640, 640)).copy()
    libc.free(out.allocated)
    return res


def ref_add_seconds(a, b, reruns: int):
    """Seconds of each of `reruns` runs of the reference's compiled add model
    (after one untimed run), the model's malloc of its output included and the
    free of it excluded: what the reference's CPU runner puts its clock around."""
    import time
    a, b = _c(a, np.float32), _c(b, np.float32)
    assert a.shape == (3, 640, 640) and b.shape == (3, 640, 640)
    ref = ctypes.CDLL(_REF_ADD_PATH)
    libc = ctypes.CDLL(None)
    libc.free.argtypes = [ctypes.c_void_p]
    descs = []
    for arr in (a, b):
        d = _MemRef3()
        d.allocated = d.aligned = arr.ctypes.data
        d.offset = 0
        d.sizes[:] = [3, 640, 640]
        d.strides[:] = [409600, 640, 1]
        descs.append(d)
    out = _MemRef3()
    times = []
    for i in range(reruns + 1):
        t0 = time.perf_counter()
        ref._mlir_ciface_main_graph(ctypes.byref(out), ctypes.byref(descs[0]), ctypes.byref(descs[1]))
        dt = time.perf_counter() - t0
        libc.free(out.allocated)
        if i:
            times.append(dt)
    return times


def _out_size(size, k, pl, pr, s, d=1):
    return (size + pl + pr - d * (k - 1) - 1) // s + 1


def conv2d(x, w, bias, post_add=None, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), relu=False):
    """NCHW fp32 cross-correlation + bias (+ post_add) (+ ReLU); pad = (top, left, bottom, right)."""
    x, w, bias, post_add = _c(x, np.float32), _c(w, np.float32), _c(bias, np.float32), _c(post_add, np.float32)
    N, IC, H, W = x.shape
    OC, IC2, KH, KW = w.shape
    assert IC == IC2 and bias.shape == (OC,)
    OH = _out_size(H, KH, pad[0], pad[2], stride[0], dilation[0])
    OW = _out_size(W, KW, pad[1], pad[3], stride[1], dilation[1])
    y = np.empty((N, OC, OH, OW), np.float32)
    i64 = ctypes.c_int64
    lib().oracle_conv2d(_p(x), _p(w), _p(bias), _p(post_add), _p(y), *[i64(v) for v in (
        N, IC, H, W, OC, KH, KW, OH, OW, pad[0], pad[1], stride[0], stride[1], dilation[0], dilation[1])],
        ctypes.c_int(1 if relu else 0))
    return y


def pool2d(x, kernel, pad=(0, 0, 0, 0), stride=(1, 1), method="max"):
    """NCHW fp32; "max" ignores the padding, "avg" divides by the full window."""
    x = _c(x, np.float32)
    N, C, H, W = x.shape
    OH = _out_size(H, kernel[0], pad[0], pad[2], stride[0])
    OW = _out_size(W, kernel[1], pad[1], pad[3], stride[1])
    y = np.empty((N, C, OH, OW), np.float32)
    i64 = ctypes.c_int64
    lib().oracle_pool2d(_p(x), _p(y), *[i64(v) for v in (
        N * C, H, W, OH, OW, kernel[0], kernel[1], pad[0], pad[1], stride[0], stride[1])],
        ctypes.c_int(0 if method == "max" else 1))
    return y
