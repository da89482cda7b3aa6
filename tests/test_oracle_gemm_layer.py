"""Pins oracle_gemm, the casts, the QKV transpose and the two layer
compositions of oracle/oracle.c against numpy / torch in fp64.  CPU only."""
import numpy as np
import torch
from scipy.special import erf


def test_gemm_against_numpy_fp64(oracle, rng):
    M, K, N = 37, 96, 50
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (0.1 * rng.standard_normal((K, N))).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16)
    r = rng.standard_normal((M, N)).astype(np.float16)
    base = x.astype(np.float64) @ w.astype(np.float64)
    assert np.abs(oracle.gemm(x, w) - base).max() < 1e-6
    assert np.abs(oracle.gemm(x, w, b) - (base + b.astype(np.float64))).max() < 1e-6
    relu = np.maximum(base + b.astype(np.float64), 0)
    assert np.abs(oracle.gemm(x, w, b, act=oracle.ACT_RELU) - relu).max() < 1e-6
    v = base + b.astype(np.float64)
    gelu = 0.5 * v * (1 + erf(v / np.sqrt(2)))
    assert np.abs(oracle.gemm(x, w, b, act=oracle.ACT_GELU) - gelu).max() < 1e-6
    tg = torch.nn.functional.gelu(torch.from_numpy(v)).numpy()  # erf form
    assert np.abs(gelu - tg).max() < 1e-12
    res = base + b.astype(np.float64) + r.astype(np.float64)
    assert np.abs(oracle.gemm(x, w, b, residual=r) - res).max() < 1e-6
    # not transposed: a non-square, non-symmetric case with a one-hot input row
    e = np.zeros((1, K), np.float16)
    e[0, 5] = 1
    assert np.array_equal(oracle.gemm(e, w)[0], w[5].astype(np.float32))
    # fp32 operands
    xf, wf = x.astype(np.float32) * 1.3, w.astype(np.float32) * 0.7
    assert np.abs(oracle.gemm(xf, wf) - xf.astype(np.float64) @ wf.astype(np.float64)).max() < 1e-6


def test_cast_matches_numpy(oracle, rng):
    f = (rng.standard_normal(200000) * np.exp(rng.uniform(-25, 12, 200000))).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16)
    assert np.array_equal(oracle.cast_f32_to_f16(f).view(np.uint16), ref.view(np.uint16))


def test_qkv_bias_transpose(oracle, rng):
    B, S, H, D = 2, 7, 3, 8
    qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float16)
    bias = rng.standard_normal((3, H, D)).astype(np.float16)
    q, k, v = oracle.qkv_bias_transpose(qkv, bias)
    s = (qkv.astype(np.float32) + bias.astype(np.float32)[None, None]).astype(np.float16).astype(np.float32)
    for i, t in enumerate((q, k, v)):
        assert np.array_equal(t, s[:, :, i].transpose(0, 2, 1, 3))


def _ln(x, g=None, b=None, eps=1e-5):
    m = x.mean(-1, keepdims=True)
    v = ((x - m) ** 2).mean(-1, keepdims=True)
    y = (x - m) / np.sqrt(v + eps)
    if g is not None:
        y = y * g + b
    return y


def _attn(qkv, H, causal, lens=None):
    B, S, _ = qkv.shape
    D = qkv.shape[-1] // 3 // H
    t = qkv.reshape(B, S, 3, H, D)
    q, k, v = [t[:, :, i].transpose(0, 2, 1, 3) for i in range(3)]
    s = q @ k.transpose(0, 1, 3, 2) / np.sqrt(D)
    mask = np.ones((B, 1, S, S), bool)
    if causal:
        mask &= np.tril(np.ones((S, S), bool))
    if lens is not None:
        for b, l in enumerate(lens):
            mask[b, :, :, l:] = False
    s = np.where(mask, s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return (p @ v).transpose(0, 2, 1, 3).reshape(B, S, H * D)


def test_decoding_context_layer_against_fp64_restatement(oracle, rng):
    """Pre-LN layer: an independent numpy fp64 restatement WITHOUT the fp16
    roundings must agree to fp16-level error, which catches a wrong op order,
    a missing residual, a wrong weight layout or mask."""
    B, S, d, ffn, H = 2, 24, 128, 256, 2
    f = lambda *s, sc=0.05: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    wqkv, wo, bo, w1, b1, w2, b2 = f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)
    for causal, act in [(True, oracle.ACT_RELU), (False, oracle.ACT_GELU)]:
        got = oracle.decoding_context_layer(x, wqkv, wo, bo, w1, b1, w2, b2, heads=H, causal=causal, act=act)
        X = x.astype(np.float64)
        a = _ln(X)
        ctx = _attn(a @ wqkv, H, causal)
        y = ctx @ wo + bo + X
        h = _ln(y) @ w1 + b1
        h = np.maximum(h, 0) if act == oracle.ACT_RELU else 0.5 * h * (1 + erf(h / np.sqrt(2)))
        ref = h @ w2 + b2 + y
        assert np.abs(got - ref).max() < 2e-2 and np.abs(got - ref).mean() < 2e-3, (causal, act)


def test_decoding_context_layer_post_ln_against_fp64_restatement(oracle, rng):
    """norm_first = false: h = LN(x + proj(attention(x))), out = LN(h + ffn(h)), identity affine.  The fp64
    restatement has no fp16 roundings; a pre-LN result, a missing residual or a LayerNorm in the wrong
    place is off by far more than the bound."""
    B, S, d, ffn, H = 2, 24, 128, 256, 2
    f = lambda *s, sc=0.05: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    wqkv, wo, bo, w1, b1, w2, b2 = f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)
    for causal, act in [(True, oracle.ACT_RELU), (False, oracle.ACT_GELU)]:
        got = oracle.decoding_context_layer(x, wqkv, wo, bo, w1, b1, w2, b2, heads=H, causal=causal, act=act,
                                            norm_first=False)
        X = x.astype(np.float64)
        h1 = _ln(_attn(X @ wqkv, H, causal) @ wo + bo + X)
        g = h1 @ w1 + b1
        g = np.maximum(g, 0) if act == oracle.ACT_RELU else 0.5 * g * (1 + erf(g / np.sqrt(2)))
        ref = _ln(g @ w2 + b2 + h1)
        assert np.abs(got - ref).max() < 2e-2 and np.abs(got - ref).mean() < 2e-3, (causal, act)
        pre = oracle.decoding_context_layer(x, wqkv, wo, bo, w1, b1, w2, b2, heads=H, causal=causal, act=act)
        assert np.abs(pre - ref).max() > 0.1  # the two orderings are far apart on these operands


def test_bert_layer_against_fp64_restatement(oracle, rng):
    B, S, d, ffn, H = 2, 20, 128, 256, 2
    h16 = lambda *s, sc=0.05: (sc * rng.standard_normal(s)).astype(np.float16)
    x = rng.standard_normal((B, S, d)).astype(np.float16)
    wqkv, bqkv, wo, bo = h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d)
    g1, be1 = (1 + h16(d).astype(np.float32)).astype(np.float16), h16(d)
    w1, b1, w2, b2 = h16(d, ffn), h16(ffn), h16(ffn, d), h16(d)
    g2, be2 = (1 + h16(d).astype(np.float32)).astype(np.float16), h16(d)
    lens = [20, 9]
    got = oracle.bert_layer_f16(x, wqkv, bqkv, wo, bo, g1, be1, w1, b1, w2, b2, g2, be2, heads=H, seqlens=lens)
    D = lambda a: a.astype(np.float64)
    X = D(x)
    ctx = _attn(X @ D(wqkv) + D(bqkv), H, False, lens)
    h1 = _ln(ctx @ D(wo) + D(bo) + X, D(g1), D(be1))
    f = h1 @ D(w1) + D(b1)
    f = 0.5 * f * (1 + erf(f / np.sqrt(2)))
    ref = _ln(f @ D(w2) + D(b2) + h1, D(g2), D(be2))
    assert np.abs(got - ref).max() < 2e-2 and np.abs(got - ref).mean() < 2e-3
