"""Parity of the HIP LayerNorm kernels (C ABI mgpuLayerNorm*, 
mgpuAddResidualPreLayerNorm*) with the oracle.

Tolerances: fp32 output |got - ref| <= 1e-5 * |ref| + 1e-6 (max relative error
1e-5 with an absolute floor at zero crossings, where a relative error is
undefined); fp16 / bf16 outputs within one unit in the last place of the
output type of the fp64 oracle value, plus 2e-6 absolute for elements where
gamma * x_hat and beta cancel (the fp32 arithmetic error of the two O(1) terms
then exceeds the spacing of fp16 near zero)."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu


def assert_f32_close(got, ref):
    err = np.abs(got - ref)
    assert np.all(err <= 1e-5 * np.abs(ref) + 1e-6), f"max abs err {err.max():.3e}"


def ulp16(ref):
    """Spacing of fp16 at |ref| (normal range)."""
    e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -14)))
    return 2.0 ** (e - 10) + 2e-6


def params(rng, n, dtype=np.float32):
    g = (1 + 0.02 * rng.standard_normal(n)).astype(dtype)
    b = (0.02 * rng.standard_normal(n)).astype(dtype)
    return g, b


def test_layernorm_config1_fp32_full_size(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20241))
    x = rng.standard_normal((32, 128, 768)).astype(np.float32)
    g, b = params(rng, 768)
    y = pkg.layer_norm(to_dev(x, gpu), to_dev(g, gpu), to_dev(b, gpu)).cpu().numpy()
    assert_f32_close(y, oracle.layernorm(x, g, b))


def test_layernorm_config1_fp16_full_size(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20241))
    x = rng.standard_normal((32, 128, 768)).astype(np.float16)
    g, b = params(rng, 768, np.float16)
    y = pkg.layer_norm(to_dev(x, gpu), to_dev(g, gpu), to_dev(b, gpu)).cpu().numpy()
    ref = oracle.layernorm(x, g, b)
    assert np.all(np.abs(y.astype(np.float32) - ref) <= ulp16(ref))
    # almost every element is the correctly rounded fp16 of the fp64 result
    assert np.mean(y == ref.astype(np.float16)) > 0.999


# one case per code path: 16-, 32- and 64-lane register kernels with full and
# partly filled lanes, the block-per-row kernel for odd, unaligned-length and
# very wide rows
@pytest.mark.parametrize("m,n", [(1, 4), (3, 64), (5, 100), (7, 256), (9, 260), (4, 512), (6, 768),
                                 (5, 1000), (3, 1024), (2, 2048), (2, 2052), (3, 4096), (2, 8200),
                                 (5, 1), (4, 2), (3, 6), (3, 7), (2, 770), (1, 12289), (1000, 96),
                                 # the block-per-row register kernel: 4 / 8 / 16 vectors per thread, full and ragged
                                 (5, 3072), (7, 4096), (3, 5000), (6, 8192), (4, 12288), (5, 16384), (2, 16388),
                                 (600, 4096)])
def test_layernorm_fp32_shapes(pkg, gpu, oracle, rng, m, n):
    x = (rng.standard_normal((m, n)) * 2 + 0.5).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    y = pkg.layer_norm(to_dev(x, gpu), to_dev(g, gpu), to_dev(b, gpu)).cpu().numpy()
    ref = oracle.layernorm(x, g, b)
    err = np.abs(y - ref)
    assert np.all(err <= 1e-5 * np.abs(ref) + 2e-6), f"max abs err {err.max():.3e}"


@pytest.mark.parametrize("m,n", [(3, 8), (4, 128), (5, 768), (2, 1000), (3, 1024), (2, 4096), (3, 8192),
                                 (2, 9), (3, 770), (2, 20000), (5, 16384), (3, 24576), (4, 32768), (2, 32776),
                                 (300, 8192)])
def test_layernorm_fp16_shapes(pkg, gpu, oracle, rng, m, n):
    x = rng.standard_normal((m, n)).astype(np.float16)
    g = rng.standard_normal(n).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float16)
    y = pkg.layer_norm(to_dev(x, gpu), to_dev(g, gpu), to_dev(b, gpu)).cpu().numpy()
    ref = oracle.layernorm(x, g, b)
    assert np.all(np.abs(y.astype(np.float32) - ref) <= ulp16(ref))


def test_layernorm_bf16(pkg, gpu, oracle, rng):
    import torch
    for m, n in [(64, 768), (3, 1000), (2, 333), (5, 8192), (3, 12288), (2, 32768)]:
        xf = rng.standard_normal((m, n)).astype(np.float32)
        gf, bf = params(rng, n)
        x, g, b = [torch.from_numpy(t).to(gpu).to(torch.bfloat16) for t in (xf, gf, bf)]
        y = pkg.layer_norm(x, g, b).float().cpu().numpy()
        bits = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)
        ref = oracle.layernorm(bits(x), bits(g), bits(b), bf16=True)
        assert np.all(np.abs(y - ref) <= np.abs(ref) * 2.0 ** -7 + 1e-6)  # one bf16 ulp


def test_add_residual_layernorm_fp16(pkg, gpu, oracle, rng):
    for m, n in [(4096, 768), (5, 1000), (3, 77), (64, 8192), (5, 12288), (3, 32768)]:
        a = rng.standard_normal((m, n)).astype(np.float16)
        r = rng.standard_normal((m, n)).astype(np.float16)
        g, b = params(rng, n, np.float16)
        s, y = pkg.add_residual_layer_norm(to_dev(a, gpu), to_dev(r, gpu), to_dev(g, gpu), to_dev(b, gpu))
        rs, ry = oracle.add_residual_layernorm(a, r, g, b)
        assert np.array_equal(s.cpu().numpy().astype(np.float32), rs)  # the rounded sum is exact
        assert np.all(np.abs(y.cpu().numpy().astype(np.float32) - ry) <= ulp16(ry))


@pytest.mark.parametrize("m,n", [(300, 768), (33, 4096), (5, 6000), (4, 16384)])
def test_add_residual_layernorm_fp32(pkg, gpu, oracle, rng, m, n):
    a = rng.standard_normal((m, n)).astype(np.float32)
    r = rng.standard_normal((m, n)).astype(np.float32)
    g, b = params(rng, n)
    s, y = pkg.add_residual_layer_norm(to_dev(a, gpu), to_dev(r, gpu), to_dev(g, gpu), to_dev(b, gpu))
    rs, ry = oracle.add_residual_layernorm(a, r, g, b)
    assert np.array_equal(s.cpu().numpy(), rs)
    assert_f32_close(y.cpu().numpy(), ry)


def test_layernorm_properties_large(pkg, gpu):
    """Size-independent properties on a matrix larger than any config
    (65536 x 1024): zero mean / unit variance for gamma = 1, beta = 0, a constant
    row maps to beta, shifting a row by a representable constant changes nothing
    beyond rounding, and the call is deterministic."""
    import torch
    g = torch.Generator(device=gpu)
    g.manual_seed(3)
    m, n = 65536, 1024
    x = torch.randn((m, n), device=gpu, generator=g)
    ones, zeros = torch.ones(n, device=gpu), torch.zeros(n, device=gpu)
    y = pkg.layer_norm(x, ones, zeros)
    assert y.mean(-1).abs().max().item() < 1e-6
    assert (y.var(-1, unbiased=False) - 1).abs().max().item() < 1e-4
    assert torch.equal(y, pkg.layer_norm(x, ones, zeros))
    beta = torch.randn(n, device=gpu, generator=g)
    c = torch.full((4, n), 2.5, device=gpu)
    assert torch.equal(pkg.layer_norm(c, ones, beta), beta.expand(4, n))
    assert (pkg.layer_norm(x[:1024] + 4.0, ones, zeros) - y[:1024]).abs().max().item() < 2e-5


def test_layernorm_in_place_and_empty(pkg, gpu, oracle, rng):
    import torch
    x = rng.standard_normal((64, 768)).astype(np.float32)
    g, b = params(rng, 768)
    t = to_dev(x, gpu)
    pkg.layer_norm(t, to_dev(g, gpu), to_dev(b, gpu), out=t)
    assert_f32_close(t.cpu().numpy(), oracle.layernorm(x, g, b))
    e = torch.empty((0, 768), device=gpu)
    assert pkg.layer_norm(e, to_dev(g, gpu), to_dev(b, gpu)).shape == (0, 768)


@pytest.mark.parametrize("m,n", [(1, 8), (5, 64), (33, 768), (100, 1000), (4096, 2048), (7, 4096), (3, 520)])
def test_cast_layer_norm_matches_cast_then_layer_norm(pkg, gpu, oracle, rng, m, n):
    """mgpuCastLayerNormF32ToF16 against mgpuCastF32ToF16 followed by mgpuLayerNormF16: the cast to the
    bit, the normalised rows to one unit in the last place (the compiler may fold the final rounding
    into the last multiply-add of one kernel and not of the other), and against the oracle like any
    fp16 LayerNorm."""
    import torch
    xh = (rng.standard_normal((m, n)) * 3 + 0.5).astype(np.float32)
    gh, bh = rng.standard_normal(n).astype(np.float16), rng.standard_normal(n).astype(np.float16)
    x, gamma, beta = to_dev(xh, gpu), to_dev(gh, gpu), to_dev(bh, gpu)
    cast, normed = pkg.cast_layer_norm(x, gamma, beta)
    ref_cast = pkg.cast_f32_to_f16(x.flatten()).view(m, n)
    ref_normed = pkg.layer_norm(ref_cast, gamma, beta)
    assert torch.equal(cast, ref_cast)
    bits = lambda t: t.view(torch.int16).cpu().numpy().astype(np.int32)
    a, b = bits(normed), bits(ref_normed)
    same_sign = (a < 0) == (b < 0)
    assert np.all(np.where(same_sign, np.abs(a - b), np.abs(a & 0x7fff) + np.abs(b & 0x7fff)) <= 1)
    want = oracle.layernorm(xh.astype(np.float16), gh, bh, 1e-5)
    got = normed.cpu().numpy().astype(np.float32)
    assert np.all(np.abs(got - want) <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -14))) - 10) + 1e-3)


def test_cast_layer_norm_refuses_other_widths(pkg, gpu):
    import torch
    for n in (12, 4104):
        x = torch.zeros((2, n), device=gpu)
        g = torch.zeros(n, device=gpu, dtype=torch.float16)
        with pytest.raises(pkg.MgpuError):
            pkg.cast_layer_norm(x, g, g)
