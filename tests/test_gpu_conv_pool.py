"""Parity of mgpuConv2d / mgpuPool2d (C ABI, NCHW fp32) with the oracle.

Pooling is exact (max) or one fp32 rounding of the window sum (average).  The
convolution accumulates fp32 products on the matrix cores in an order of its
own (true fp32 products, unlike the reduced-precision ones the reference
allows through CUDNN_TENSOR_OP_MATH_ALLOW_CONVERSION): the bound is
1e-4 (1 + |ref|), checked elementwise."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu


def conv_case(pkg, gpu, oracle, rng, N, IC, H, W, OC, K, pad, stride, dilation, relu, add):
    x = rng.standard_normal((N, IC, H, W)).astype(np.float32)
    w = (rng.standard_normal((OC, IC) + K) / np.sqrt(IC * K[0] * K[1])).astype(np.float32)
    b = rng.standard_normal(OC).astype(np.float32)
    ref = oracle.conv2d(x, w, b, None, pad, stride, dilation, False)
    a = rng.standard_normal(ref.shape).astype(np.float32) if add else None
    ref = oracle.conv2d(x, w, b, a, pad, stride, dilation, relu)
    got = pkg.conv2d(to_dev(x, gpu), to_dev(w, gpu), to_dev(b, gpu), to_dev(a, gpu) if add else None,
                     pad, stride, dilation, relu).cpu().numpy()
    assert got.shape == ref.shape
    err = np.abs(got - ref)
    assert np.all(err <= 1e-4 * (1.0 + np.abs(ref))), err.max()
    return err.max()


@pytest.mark.parametrize("N,IC,H,W,OC,K,pad,stride,dilation,relu,add", [
    (2, 3, 9, 11, 4, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), False, False),
    (1, 4, 12, 10, 5, (3, 2), (0, 1, 2, 0), (2, 1), (1, 1), True, True),    # asymmetric padding
    (2, 2, 15, 15, 3, (3, 3), (2, 2, 2, 2), (2, 2), (2, 2), True, False),    # dilation
    (3, 8, 7, 7, 6, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), False, True),      # pointwise
    (1, 1, 5, 5, 1, (5, 5), (0, 0, 0, 0), (1, 1), (1, 1), False, False),     # one output element
    (2, 3, 64, 64, 16, (7, 7), (3, 3, 3, 3), (2, 2), (1, 1), True, False),   # ResNet stem, scaled down
    (4, 64, 28, 28, 64, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), True, True),   # ResNet basic block conv + shortcut
    (4, 256, 14, 14, 64, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), True, False), # bottleneck reduce
    (2, 64, 28, 28, 128, (1, 1), (0, 0, 0, 0), (2, 2), (1, 1), False, False),# strided pointwise (downsample)
])
def test_conv2d(pkg, gpu, oracle, rng, N, IC, H, W, OC, K, pad, stride, dilation, relu, add):
    conv_case(pkg, gpu, oracle, rng, N, IC, H, W, OC, K, pad, stride, dilation, relu, add)


@pytest.mark.parametrize("C,H,W,K,pad,stride", [
    (3, 8, 8, (2, 2), (0, 0, 0, 0), (2, 2)), (2, 9, 7, (3, 3), (1, 1, 1, 1), (2, 2)),
    (64, 112, 112, (3, 3), (1, 1, 1, 1), (2, 2)),  # ResNet stem pool
    (512, 7, 7, (7, 7), (0, 0, 0, 0), (1, 1)),     # global average pool
    (2, 10, 11, (3, 2), (1, 0, 1, 1), (2, 1)),
])
def test_pool2d(pkg, gpu, oracle, rng, C, H, W, K, pad, stride):
    x = rng.standard_normal((2, C, H, W)).astype(np.float32)
    tx = to_dev(x, gpu)
    assert np.array_equal(pkg.pool2d(tx, K, pad, stride, "max").cpu().numpy(), oracle.pool2d(x, K, pad, stride, "max"))
    avg, ref = pkg.pool2d(tx, K, pad, stride, "avg").cpu().numpy(), oracle.pool2d(x, K, pad, stride, "avg")
    assert np.all(np.abs(avg - ref) <= 1e-6 * (1 + np.abs(ref)))


def test_conv_pool_reject_bad_arguments(pkg, gpu):
    import torch
    x = torch.zeros((1, 2, 8, 8), device=gpu)
    w = torch.zeros((3, 2, 3, 3), device=gpu)
    b = torch.zeros(3, device=gpu)
    lib = pkg.ops()
    out = torch.zeros((1, 3, 8, 8), device=gpu)
    args = lambda OH: (x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), None, 1, 2, 8, 8, 3, 3, 3, OH, 8,
                       1, 1, 1, 1, 1, 1, 1, 1, False, False, None)
    lib.mgpuConv2d(*args(7))
    assert b"output size does not follow" in lib.mgpuOpsTakeLastError()
    lib.mgpuConv2d(*args(8)[:4], None, *args(8)[5:22], True, False, None)
    assert b"hasPostAdd" in lib.mgpuOpsTakeLastError()
    lib.mgpuPool2d(x.data_ptr(), out.data_ptr(), 1, 2, 8, 8, 4, 4, 2, 2, 0, 0, 0, 0, 2, 2, 5, None)
    assert b"method" in lib.mgpuOpsTakeLastError()
    lib.mgpuPool2d(x.data_ptr(), out.data_ptr(), 1, 2, 8, 8, 5, 5, 2, 2, 2, 2, 0, 0, 2, 2, 0, None)
    assert b"padding must be smaller" in lib.mgpuOpsTakeLastError()
    assert lib.mgpuOpsTakeLastError() is None
