"""Pins of the oracle's convolution and pooling (CPU): torch's CPU conv2d /
max_pool2d / avg_pool2d in fp64, hand-computed tiny cases, and the identities a
dropped term or a transposed index would break."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F


def torch_conv(x, w, b, add, pad, stride, dilation, relu):
    xt = F.pad(torch.from_numpy(x).double(), (pad[1], pad[3], pad[0], pad[2]))
    y = F.conv2d(xt, torch.from_numpy(w).double(), torch.from_numpy(b).double(), stride=stride, dilation=dilation)
    if add is not None:
        y = y + torch.from_numpy(add).double()
    if relu:
        y = torch.relu(y)
    return y.numpy()


@pytest.mark.parametrize("N,IC,H,W,OC,K,pad,stride,dilation,relu,add", [
    (2, 3, 9, 11, 4, (3, 3), (1, 1, 1, 1), (1, 1), (1, 1), False, False),
    (1, 4, 12, 10, 5, (3, 2), (0, 1, 2, 0), (2, 1), (1, 1), True, True),   # asymmetric padding
    (2, 2, 15, 15, 3, (3, 3), (2, 2, 2, 2), (2, 2), (2, 2), True, False),   # dilation
    (3, 8, 7, 7, 6, (1, 1), (0, 0, 0, 0), (1, 1), (1, 1), False, True),     # pointwise
    (1, 1, 5, 5, 1, (5, 5), (0, 0, 0, 0), (1, 1), (1, 1), False, False),    # one output element
    (1, 3, 16, 16, 2, (7, 7), (3, 3, 3, 3), (2, 2), (1, 1), True, False),
])
def test_conv2d_against_torch(oracle, rng, N, IC, H, W, OC, K, pad, stride, dilation, relu, add):
    x = rng.standard_normal((N, IC, H, W)).astype(np.float32)
    w = rng.standard_normal((OC, IC) + K).astype(np.float32)
    b = rng.standard_normal(OC).astype(np.float32)
    got = oracle.conv2d(x, w, b, None, pad, stride, dilation, relu)
    a = rng.standard_normal(got.shape).astype(np.float32) if add else None
    got = oracle.conv2d(x, w, b, a, pad, stride, dilation, relu)
    ref = torch_conv(x, w, b, a, pad, stride, dilation, relu)
    assert got.shape == ref.shape
    assert np.abs(got - ref).max() <= 1e-6 * max(1.0, np.abs(ref).max())


def test_conv2d_by_hand_and_orientation(oracle):
    # a single 1 in the image copies the filter, un-flipped for cross-correlation:
    # y[oh, ow] = w[2 - oh, 2 - ow] when the 1 sits at (2, 2) of a 5x5 image (3x3 filter, no padding)
    x = np.zeros((1, 1, 5, 5), np.float32)
    x[0, 0, 2, 2] = 1
    w = np.arange(9, dtype=np.float32).reshape(1, 1, 3, 3)
    y = oracle.conv2d(x, w, np.zeros(1, np.float32))
    assert np.array_equal(y[0, 0], w[0, 0, ::-1, ::-1])
    # bias only, then ReLU and post-add
    z = np.zeros((1, 2, 4, 4), np.float32)
    w2 = np.ones((3, 2, 3, 3), np.float32)
    b = np.array([-1.0, 0.5, 2.0], np.float32)
    y = oracle.conv2d(z, w2, b, None, (1, 1, 1, 1), relu=True)
    assert np.array_equal(y, np.broadcast_to(np.array([0, 0.5, 2.0], np.float32)[None, :, None, None], (1, 3, 4, 4)))
    add = np.full((1, 3, 4, 4), 0.75, np.float32)
    y = oracle.conv2d(z, w2, b, add, (1, 1, 1, 1), relu=True)
    assert np.array_equal(y[0, :, 0, 0], np.array([0.0, 1.25, 2.75], np.float32))
    # all-ones 3x3 filter with padding 1 counts the neighbours inside the image
    ones = np.ones((1, 1, 3, 3), np.float32)
    y = oracle.conv2d(ones, np.ones((1, 1, 3, 3), np.float32), np.zeros(1, np.float32), None, (1, 1, 1, 1))
    assert np.array_equal(y[0, 0], np.array([[4, 6, 4], [6, 9, 6], [4, 6, 4]], np.float32))


def test_conv2d_linearity(oracle, rng):
    x1, x2 = rng.standard_normal((2, 1, 3, 8, 8)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    z = np.zeros(4, np.float32)
    lhs = oracle.conv2d(x1 + x2, w, z, None, (1, 1, 1, 1))
    rhs = oracle.conv2d(x1, w, z, None, (1, 1, 1, 1)) + oracle.conv2d(x2, w, z, None, (1, 1, 1, 1))
    assert np.abs(lhs - rhs).max() <= 1e-5


@pytest.mark.parametrize("C,H,W,K,pad,stride", [
    (3, 8, 8, (2, 2), (0, 0, 0, 0), (2, 2)), (2, 9, 7, (3, 3), (1, 1, 1, 1), (2, 2)),
    (4, 12, 12, (3, 3), (1, 1, 1, 1), (1, 1)), (1, 7, 7, (7, 7), (0, 0, 0, 0), (1, 1)),
    (2, 10, 11, (3, 2), (1, 0, 1, 1), (2, 1)),
])
def test_pool2d_against_torch(oracle, rng, C, H, W, K, pad, stride):
    x = rng.standard_normal((2, C, H, W)).astype(np.float32)
    xt = torch.from_numpy(x).double()
    neg = F.pad(xt, (pad[1], pad[3], pad[0], pad[2]), value=float("-inf"))
    zero = F.pad(xt, (pad[1], pad[3], pad[0], pad[2]))
    ref_max = F.max_pool2d(neg, K, stride).numpy()
    ref_avg = F.avg_pool2d(zero, K, stride).numpy()  # zeros of the padding are counted
    assert np.array_equal(oracle.pool2d(x, K, pad, stride, "max"), ref_max.astype(np.float32))
    assert np.abs(oracle.pool2d(x, K, pad, stride, "avg") - ref_avg).max() <= 1e-6


def test_pool2d_by_hand(oracle):
    x = np.arange(16, dtype=np.float32).reshape(1, 1, 4, 4)
    assert np.array_equal(oracle.pool2d(x, (2, 2), stride=(2, 2))[0, 0], np.array([[5, 7], [13, 15]], np.float32))
    assert np.array_equal(oracle.pool2d(x, (2, 2), stride=(2, 2), method="avg")[0, 0],
                          np.array([[2.5, 4.5], [10.5, 12.5]], np.float32))
    # padded corner: max ignores the padding, the average divides by the full window
    neg = -np.ones((1, 1, 2, 2), np.float32)
    assert oracle.pool2d(neg, (2, 2), (1, 1, 1, 1), (2, 2))[0, 0, 0, 0] == -1
    assert oracle.pool2d(neg, (2, 2), (1, 1, 1, 1), (2, 2), "avg")[0, 0, 0, 0] == -0.25
