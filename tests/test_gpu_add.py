"""Parity of the HIP elementwise add (C ABI mgpuAddF32) with the oracle and the
reference's golden vectors: bit exact."""
import os

import numpy as np
import pytest

from conftest import GOLDEN, to_dev

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def same(x, y):
    return np.all((bits(x) == bits(y)) | (np.isnan(x) & np.isnan(y)))


def test_add_config0_full_size_bit_exact(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20240))
    a = rng.uniform(-1, 1, (3, 640, 640)).astype(np.float32)
    b = rng.uniform(-1, 1, (3, 640, 640)).astype(np.float32)
    c = pkg.add(to_dev(a, gpu), to_dev(b, gpu)).cpu().numpy()
    assert np.array_equal(bits(c), bits(oracle.add_f32(a, b)))


def test_add_reference_golden_vectors(pkg, gpu):
    """Inputs and outputs recorded from the reference's compiled add model,
    including NaN, +-Inf, signed zeros, denormals and rounding cases."""
    g = np.load(os.path.join(GOLDEN, "add_ref_3x640x640_sample.npz"))
    a, b = g["a_bits"].view(np.float32), g["b_bits"].view(np.float32)
    c = pkg.add(to_dev(a, gpu), to_dev(b, gpu)).cpu().numpy()
    assert same(c, g["c_bits"].view(np.float32))
    assert c[9] != 0  # denormal sum survives: no flush to zero


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 255, 256, 257, 1023, 4097, 100003, 2 ** 20 + 1])
def test_add_ragged_sizes(pkg, gpu, oracle, rng, n):
    a = (rng.standard_normal(n) * np.exp(rng.uniform(-40, 40, n))).astype(np.float32)
    b = (rng.standard_normal(n) * np.exp(rng.uniform(-40, 40, n))).astype(np.float32)
    c = pkg.add(to_dev(a, gpu), to_dev(b, gpu)).cpu().numpy()
    assert np.array_equal(bits(c), bits(oracle.add_f32(a, b)))


def test_add_unaligned_pointers_take_the_scalar_path(pkg, gpu, oracle, rng):
    import torch
    n = 10001
    a = rng.standard_normal(n + 3).astype(np.float32)
    b = rng.standard_normal(n + 3).astype(np.float32)
    ta, tb = to_dev(a, gpu), to_dev(b, gpu)
    out = torch.zeros(n + 3, device=gpu)
    for off in (1, 2, 3):
        pkg.add(ta[off:off + n], tb[off:off + n], out[off:off + n])
        assert np.array_equal(out[off:off + n].cpu().numpy(), oracle.add_f32(a[off:off + n], b[off:off + n]))
    # nothing outside the requested range is written
    out.zero_()
    pkg.add(ta[1:n], tb[1:n], out[1:n])
    assert out[0].item() == 0 and out[n:].abs().sum().item() == 0


def test_add_large_and_properties(pkg, gpu, rng):
    """Bigger than any config (64 Mi elements): commutativity and a + 0 = a
    hold bit for bit, and the result equals the fp64 sum rounded once."""
    import torch
    n = 1 << 26
    g = torch.Generator(device=gpu)
    g.manual_seed(5)
    a = torch.randn(n, device=gpu, generator=g) * 1e3
    b = torch.randn(n, device=gpu, generator=g)
    c = pkg.add(a, b)
    assert torch.equal(c.view(torch.int32), pkg.add(b, a).view(torch.int32))
    assert torch.equal(pkg.add(a, torch.zeros_like(a)).view(torch.int32), a.view(torch.int32))
    exact = (a.double() + b.double()).float()
    assert torch.equal(c.view(torch.int32), exact.view(torch.int32))


def test_add_beyond_the_grid_cap(pkg, gpu):
    """The launch is capped at 2^22 blocks; beyond 2^32 + 1024 elements on the vector path (2^30 on the scalar
    path, which unaligned pointers take) a block walks on by the size of the grid.  Checked on the device against
    the fp64 sum rounded once, a slice at a time; 52 GB of device memory."""
    import torch
    n = (1 << 32) + 4 * 256 * 3 + 7
    if torch.cuda.mem_get_info(gpu)[0] < 60 * (1 << 30):
        pytest.skip("needs 60 GB of free device memory")
    a = torch.empty(n, device=gpu).uniform_(-1e3, 1e3)
    b = torch.empty(n, device=gpu).uniform_(-1.0, 1.0)
    c = torch.zeros(n + 8, device=gpu)

    def same(lo, hi, shift=0):
        step = 1 << 28
        for i in range(lo, hi, step):
            j = min(hi, i + step)
            exact = (a[i:j].double() + b[i:j].double()).float()
            if not torch.equal(c[i + shift:j + shift].view(torch.int32), exact.view(torch.int32)):
                return False
        return True

    pkg.add(a, b, out=c[:n])
    assert same(0, n) and c[n:].abs().sum().item() == 0
    # the scalar path: every pointer one element off 16-byte alignment
    m = (1 << 30) + 5
    c.zero_()
    pkg.add(a[1:1 + m], b[1:1 + m], out=c[1:1 + m])
    assert same(1, 1 + m) and c[0].item() == 0 and c[1 + m:1 + m + 1024].abs().sum().item() == 0


def test_add_empty(pkg, gpu):
    import torch
    e = torch.empty(0, device=gpu)
    assert pkg.add(e, e).numel() == 0
