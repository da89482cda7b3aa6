"""Pins oracle_layernorm / oracle_add_residual_layernorm / the 16-bit
conversions of oracle/oracle.c.  CPU only."""
import numpy as np
import torch


def test_half_conversions_exhaustive(oracle):
    allh = np.arange(65536, dtype=np.uint16)
    f = oracle.half_to_float(allh)
    ref = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(f.view(np.uint32), ref.view(np.uint32))
    # every half value round-trips through the double -> half conversion
    back = oracle.double_to_half(f.astype(np.float64)).view(np.uint16)
    nan = np.isnan(ref)
    assert np.array_equal(back[~nan], allh[~nan]) and np.all(np.isnan(back[nan].view(np.float16)))


def test_double_to_half_rounding(oracle, rng):
    d = rng.standard_normal(400000) * np.exp(rng.uniform(-22, 12, 400000))
    with np.errstate(over="ignore"):
        ref = d.astype(np.float16)
    assert np.array_equal(oracle.double_to_half(d).view(np.uint16), ref.view(np.uint16))
    # exact halfway cases between neighbouring halves must go to even
    h = rng.integers(0x0001, 0x7bfe, 20000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = (lo + hi) / 2
    got = oracle.double_to_half(mid).view(np.uint16)
    assert np.array_equal(got, np.where(h % 2 == 0, h, h + 1))
    # a double that fp32 would round onto the halfway point first (double rounding trap)
    x = np.array([1.0 + 2.0 ** -11 + 2.0 ** -40], np.float64)
    assert oracle.double_to_half(x).view(np.uint16)[0] == 0x3c01


def test_bf16_conversions(oracle, rng):
    f = (rng.standard_normal(100000) * np.exp(rng.uniform(-30, 30, 100000))).astype(np.float32)
    ref = torch.from_numpy(f).to(torch.bfloat16)
    got = oracle.float_to_bf16(f)
    assert np.array_equal(got, ref.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(oracle.bf16_to_float(got), ref.float().numpy())


def test_layernorm_against_torch_fp64(oracle, rng):
    for (m, n) in [(7, 768), (3, 5), (1, 1024), (16, 33)]:
        x = rng.standard_normal((m, n)).astype(np.float32) * 3 + 1
        g = (1 + 0.02 * rng.standard_normal(n)).astype(np.float32)
        b = (0.02 * rng.standard_normal(n)).astype(np.float32)
        ref = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (n,), torch.from_numpy(g).double(),
                                             torch.from_numpy(b).double(), 1e-5).numpy()
        got = oracle.layernorm(x, g, b, 1e-5)
        assert np.abs(got - ref).max() <= 4e-7 * max(1.0, np.abs(ref).max())


def test_layernorm_hand_computed_rows(oracle):
    # n = 2: x = (a, b) -> mean (a+b)/2, var ((a-b)/2)^2 ; with eps = 0 the
    # normalised row is (+-1) whatever a, b are.
    x = np.array([[3.0, 7.0], [-2.0, -10.0]], np.float32)
    y = oracle.layernorm(x, np.ones(2, np.float32), np.zeros(2, np.float32), eps=0.0)
    assert np.allclose(y, [[-1, 1], [1, -1]], atol=1e-7)
    # n = 4: x = (1,2,3,4): mean 2.5, biased var 1.25
    x = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    y = oracle.layernorm(x, np.full(4, 2.0, np.float32), np.full(4, 0.5, np.float32), eps=0.0)
    assert np.allclose(y, (x - 2.5) / np.sqrt(1.25) * 2 + 0.5, atol=1e-7)
    # eps enters inside the square root: var = 0 row with eps = 0.25 -> (x-mean)/0.5 = 0
    # and a var = 0.75 row with eps 0.25 divides by exactly 1
    x = np.array([[0.0, 0.0, 2.0, 2.0, 1.0, 1.0]], np.float32)  # mean 1, var 4/6
    y = oracle.layernorm(x, np.ones(6, np.float32), np.zeros(6, np.float32), eps=1.0 / 3.0)
    assert np.allclose(y, x - 1.0, atol=1e-7)
    # biased (1/n), not unbiased (1/(n-1)) variance
    x = np.array([[0.0, 2.0]], np.float32)  # biased var 1 -> y = +-1 ; unbiased var 2 -> +-0.707
    y = oracle.layernorm(x, np.ones(2, np.float32), np.zeros(2, np.float32), eps=0.0)
    assert np.allclose(np.abs(y), 1.0, atol=1e-7)


def test_layernorm_identities(oracle, rng):
    n = 96
    x = rng.standard_normal((5, n)).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32)
    y = oracle.layernorm(x, g, b)
    # constant row -> beta
    c = np.full((1, n), 3.25, np.float32)
    assert np.allclose(oracle.layernorm(c, g, b), b, atol=1e-6)
    # shift invariance (shift exactly representable)
    assert np.allclose(oracle.layernorm(x + np.float32(8.0), g, b), y, atol=2e-5)
    # gamma = 1, beta = 0: zero mean, unit variance (up to eps)
    z = oracle.layernorm(x, np.ones(n, np.float32), np.zeros(n, np.float32))
    assert np.abs(z.mean(-1)).max() < 1e-6 and np.abs(z.var(-1) - 1).max() < 1e-4
    # null gamma/beta mean 1/0
    assert np.array_equal(oracle.layernorm(x, None, None), z)


def test_layernorm_fp16_inputs_use_the_rounded_values(oracle, rng):
    x = rng.standard_normal((4, 64)).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(64)).astype(np.float16)
    b = (0.1 * rng.standard_normal(64)).astype(np.float16)
    got = oracle.layernorm(x, g, b)
    ref = oracle.layernorm(x.astype(np.float32), g.astype(np.float32), b.astype(np.float32))
    assert np.array_equal(got, ref)


def test_add_residual_layernorm(oracle, rng):
    m, n = 6, 128
    a = rng.standard_normal((m, n)).astype(np.float16)
    r = rng.standard_normal((m, n)).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(n)).astype(np.float16)
    b = (0.1 * rng.standard_normal(n)).astype(np.float16)
    s, y = oracle.add_residual_layernorm(a, r, g, b)
    # the stored sum is fp16(fp32(a) + fp32(r))
    s_ref = (a.astype(np.float32) + r.astype(np.float32)).astype(np.float16)
    assert np.array_equal(s, s_ref.astype(np.float32))
    # statistics from the un-rounded sums, normalised value from the rounded sum
    s32 = (a.astype(np.float32) + r.astype(np.float32)).astype(np.float64)
    mean = s32.mean(-1, keepdims=True)
    var = ((s32 - mean) ** 2).mean(-1, keepdims=True)
    y_ref = (s_ref.astype(np.float64) - mean) / np.sqrt(var + 1e-5) * g.astype(np.float64) + b.astype(np.float64)
    assert np.abs(y - y_ref).max() < 1e-6
    # residual == 0 reduces to plain LayerNorm
    z = np.zeros_like(a)
    s0, y0 = oracle.add_residual_layernorm(a, z, g, b)
    assert np.array_equal(s0, a.astype(np.float32))
    assert np.array_equal(y0, oracle.layernorm(a, g, b))
    # fp32: sum is not re-rounded
    a32, r32 = a.astype(np.float32) * 1.37, r.astype(np.float32) * 0.77
    s1, _ = oracle.add_residual_layernorm(a32, r32, g.astype(np.float32), b.astype(np.float32))
    assert np.array_equal(s1, a32 + r32)
