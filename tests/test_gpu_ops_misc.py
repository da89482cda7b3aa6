"""Casts, QKV bias+transpose, GEMM epilogues and the two layer entry points
against the oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 7, 8, 9, 1000, 65537, 3 * 768 * 768])
def test_casts_bit_exact(pkg, gpu, oracle, rng, n):
    f = (rng.standard_normal(n) * np.exp(rng.uniform(-20, 12, n))).astype(np.float32)
    h = pkg.cast_f32_to_f16(to_dev(f, gpu))
    assert np.array_equal(h.cpu().numpy().view(np.uint16), oracle.cast_f32_to_f16(f).view(np.uint16))
    back = pkg.cast_f16_to_f32(h).cpu().numpy()
    assert np.array_equal(back.view(np.uint32), oracle.half_to_float(h.cpu().numpy()).view(np.uint32))


def test_cast_special_values(pkg, gpu, oracle):
    f = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65520.0, 65519.9, 1e-8, 5.96e-8, 2.98e-8,
                  2.99e-8, 6.1e-5, 1.0 + 2 ** -11, 1.0 + 2 ** -11 + 2 ** -20, 1.0 + 3 * 2 ** -11], np.float32)
    h = pkg.cast_f32_to_f16(to_dev(f, gpu)).cpu().numpy()
    ref = oracle.cast_f32_to_f16(f)
    assert np.all((h.view(np.uint16) == ref.view(np.uint16)) | (np.isnan(h) & np.isnan(ref)))


def test_qkv_bias_transpose(pkg, gpu, oracle, rng):
    B, S, H, D = 3, 50, 4, 64
    qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float16)
    bias = rng.standard_normal((3, H, D)).astype(np.float16)
    t = to_dev(qkv, gpu)
    q, k, v = pkg.qkv_bias_transpose(t, to_dev(bias, gpu))
    rq, rk, rv = oracle.qkv_bias_transpose(qkv, bias)
    for got, ref in ((q, rq), (k, rk), (v, rv)):
        assert np.array_equal(got.cpu().numpy().astype(np.float32), ref)
    # the packed tensor is updated in place with the bias, like the reference kernel
    upd = (qkv.astype(np.float32) + bias.astype(np.float32)[None, None]).astype(np.float16)
    assert np.array_equal(t.cpu().numpy(), upd)


def f16_tol(ref, k_ulp=1.0, floor=1e-3):
    e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -14)))
    return k_ulp * 2.0 ** (e - 10) + floor


@pytest.mark.parametrize("M,K,N", [(512, 768, 2304), (100, 64, 72), (4096, 3072, 768), (33, 128, 8)])
def test_matmul_ex_f16_epilogues(pkg, gpu, oracle, rng, M, K, N):
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16)
    r = rng.standard_normal((M, N)).astype(np.float16)
    tx, tw, tb, tr = [to_dev(t, gpu) for t in (x, w, b, r)]
    for kw, okw in [(dict(), dict()), (dict(bias=tb), dict(bias=b)),
                    (dict(bias=tb, act=pkg.ACT_RELU), dict(bias=b, act=oracle.ACT_RELU)),
                    (dict(bias=tb, act=pkg.ACT_GELU), dict(bias=b, act=oracle.ACT_GELU)),
                    (dict(bias=tb, residual=tr), dict(bias=b, residual=r))]:
        got = pkg.matmul_ex(tx, tw, **kw).cpu().numpy().astype(np.float32)
        ref = oracle.gemm(x, w, **okw)
        # GELU runs on the fp16-rounded GEMM output: two roundings, and the first is taken
        # at the pre-activation magnitude, which can sit one binade above the result
        k_ulp = 2.5 if kw.get("act") == pkg.ACT_GELU else 1.0
        assert np.all(np.abs(got - ref) <= f16_tol(ref, k_ulp)), (kw.keys(), np.abs(got - ref).max())


@pytest.mark.parametrize("M,K,N", [(512, 768, 2304), (100, 64, 72), (33, 130, 8)])
def test_matmul_ex_packed_weight(pkg, gpu, oracle, rng, M, K, N):
    """mgpuPackWeight16 + mgpuMatmulExPackedF16: the weight transposed once, bit for bit (odd sizes included), and
    every epilogue on the packed copy against the oracle, to the bound of the unpacked entry point."""
    import torch
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    w[0, 0], w[-1, -1] = np.float16(np.nan), np.float16(6e-8)          # a NaN and a subnormal travel unchanged
    b = rng.standard_normal(N).astype(np.float16)
    r = rng.standard_normal((M, N)).astype(np.float16)
    tx, tw, tb, tr = [to_dev(t, gpu) for t in (x, w, b, r)]
    packed = pkg.pack_weight(tw)
    assert np.array_equal(packed.cpu().numpy().view(np.uint16), np.ascontiguousarray(w.T).view(np.uint16))
    w[0, 0] = 0
    tw = to_dev(w, gpu)
    packed = pkg.pack_weight(tw)
    for kw, okw in [(dict(), dict()), (dict(bias=tb), dict(bias=b)),
                    (dict(bias=tb, act=pkg.ACT_RELU), dict(bias=b, act=oracle.ACT_RELU)),
                    (dict(bias=tb, act=pkg.ACT_GELU), dict(bias=b, act=oracle.ACT_GELU)),
                    (dict(bias=tb, residual=tr), dict(bias=b, residual=r))]:
        got = pkg.matmul_ex(tx, packed, kernel="packed", **kw).cpu().numpy().astype(np.float32)
        ref = oracle.gemm(x, w, **okw)
        k_ulp = 2.5 if kw.get("act") == pkg.ACT_GELU else 1.0
        assert np.all(np.abs(got - ref) <= f16_tol(ref, k_ulp)), (kw.keys(), np.abs(got - ref).max())
    # bf16 through the same entry points
    xb, wb = torch.randn((64, 96), device=gpu).bfloat16(), (torch.randn((96, 40), device=gpu) / 10).bfloat16()
    got = pkg.matmul_ex(xb, pkg.pack_weight(wb), kernel="packed").float()
    assert torch.allclose(got, pkg.matmul_ex(xb, wb).float(), atol=4e-2, rtol=2e-2)
    assert torch.allclose(got, xb.float() @ wb.float(), atol=4e-2, rtol=2e-2)


def bf16_bits(t):
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("n", [1, 7, 8, 9, 1000, 65537])
def test_bf16_casts_bit_exact(pkg, gpu, oracle, rng, n):
    """fp32 <-> bf16: round to nearest even on the upper 16 bits, NaN stays NaN."""
    f = (rng.standard_normal(n) * np.exp(rng.uniform(-60, 60, n))).astype(np.float32)
    if n >= 9:
        f[:9] = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 3.3895e38, 1e-40]
    h = pkg.cast_f32_to_bf16(to_dev(f, gpu))
    got, ref = bf16_bits(h), oracle.float_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], ref[~nan])
    assert np.all((got[nan] & 0x7f80) == 0x7f80) and np.all((got[nan] & 0x7f) != 0)
    back = pkg.cast_bf16_to_f32(h).cpu().numpy()
    assert np.array_equal(back.view(np.uint32), oracle.bf16_to_float(got).view(np.uint32))
    # independent pin: the upper half of the fp32 pattern, plus the closed-form rounding
    u = f[~nan].view(np.uint32).astype(np.uint64)
    assert np.array_equal(ref[~nan], ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16))


def test_qkv_bias_transpose_bf16(pkg, gpu, oracle, rng):
    import torch
    B, S, H, D = 2, 37, 3, 64
    qkv = torch.from_numpy(rng.standard_normal((B, S, 3, H, D)).astype(np.float32)).to(gpu).to(torch.bfloat16)
    bias = torch.from_numpy(rng.standard_normal((3, H, D)).astype(np.float32)).to(gpu).to(torch.bfloat16)
    qb, bb = bf16_bits(qkv), bf16_bits(bias)
    q, k, v = pkg.qkv_bias_transpose(qkv, bias)
    rq, rk, rv = oracle.qkv_bias_transpose(qb, bb, bf16=True)
    for got, ref in ((q, rq), (k, rk), (v, rv)):
        assert np.array_equal(got.float().cpu().numpy(), ref)
    upd = oracle.float_to_bf16(oracle.bf16_to_float(qb) + oracle.bf16_to_float(bb)[None, None])
    assert np.array_equal(bf16_bits(qkv), upd)


@pytest.mark.parametrize("M,K,N", [(256, 768, 768), (100, 64, 72)])
def test_matmul_ex_bf16_epilogues(pkg, gpu, oracle, rng, M, K, N):
    import torch
    mk = lambda a: torch.from_numpy(a.astype(np.float32)).to(gpu).to(torch.bfloat16)
    tx, tw = mk(rng.standard_normal((M, K))), mk(rng.standard_normal((K, N)) / np.sqrt(K))
    tb, tr = mk(rng.standard_normal(N)), mk(rng.standard_normal((M, N)))
    x, w, b, r = [bf16_bits(t) for t in (tx, tw, tb, tr)]
    for kw, okw in [(dict(), dict()), (dict(bias=tb), dict(bias=b)),
                    (dict(bias=tb, act=pkg.ACT_RELU), dict(bias=b, act=oracle.ACT_RELU)),
                    (dict(bias=tb, act=pkg.ACT_GELU), dict(bias=b, act=oracle.ACT_GELU)),
                    (dict(bias=tb, residual=tr), dict(bias=b, residual=r))]:
        got = pkg.matmul_ex(tx, tw, **kw).float().cpu().numpy()
        ref = oracle.gemm(x, w, bf16=True, **okw)
        # one bf16 spacing of the result (2^-7 relative); GELU rounds twice
        k_ulp = 2.5 if kw.get("act") == pkg.ACT_GELU else 1.0
        tol = k_ulp * 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -14))) - 7) + 4e-3
        assert np.all(np.abs(got - ref) <= tol), (kw.keys(), np.abs(got - ref).max())

@pytest.mark.parametrize("M,K,N,bound", [(200, 96, 130, 6e-6), (64, 3072, 128, 1.2e-5)])
def test_matmul_f32(pkg, gpu, oracle, rng, M, K, N, bound):
    """mgpuMatmul / mgpuMatmulExF32 run true fp32 products with fp32 accumulation (the
    reference asks cuBLASLt for CUBLAS_COMPUTE_32F_FAST_16F, Ops.cu:57-120: fp16 products).
    Measured against the fp64 oracle: max abs 1.4e-6 at K = 96, 2.9e-6 at K = 3072 for
    O(1) results; the bound is four times that, far below what fp16 or xf32 products
    give (1e-3), and a lost bias (O(1)) or a lost bias column cannot hide under it."""
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    got = pkg.matmul_ex(to_dev(x, gpu), to_dev(w, gpu), to_dev(b, gpu)).cpu().numpy()
    ref = oracle.gemm(x, w, b)
    assert np.abs(got - ref).max() <= bound
    assert np.abs(got - ref).mean() <= bound / 8


def layer_tol(ref):
    """fp16 output of an O(1..4)-magnitude tensor after ~6 fp16-rounded stages.  The floor is
    one fp16 spacing of the residual stream (2^-8 for |x| in [4, 8)): an intermediate rounded
    the other way survives into an output that the last addition brings close to zero."""
    return 5e-3 + 4e-3 * np.abs(ref)


def test_bert_encoder_layer_config4(pkg, gpu, oracle):
    """BERT-base layer (32,128,768) fp16, weights N(0, 0.02): post-LN ordering
    and erf-GELU are defined by the benchmark configuration, not by the
    reference (whose layer is pre-LN / ReLU / causal)."""
    rng = np.random.Generator(np.random.PCG64(20245))
    B, S, d, ffn, H = 32, 128, 768, 3072, 12
    h16 = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float16)
    gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
    x = rng.standard_normal((B, S, d)).astype(np.float16)
    P = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
         h16(d), gam(), h16(d)]
    for lens in (None, rng.integers(1, 129, B).astype(np.int32)):
        tl = to_dev(lens, gpu) if lens is not None else None
        got = pkg.bert_encoder_layer(to_dev(x, gpu), *[to_dev(p, gpu) for p in P], heads=H, seqlens=tl)
        got = got.cpu().numpy().astype(np.float32)
        ref = oracle.bert_layer_f16(x, *P, heads=H, seqlens=lens)
        err = np.abs(got - ref)
        assert np.all(err <= layer_tol(ref)), err.max()
        assert err.mean() <= 5e-4


def test_weight_cache_shared_by_two_streams(pkg, gpu, rng):
    """The cache is per process, not per stream: a call on one stream fills it (the conversions run on that stream's
    side stream) and a call issued right behind it on another stream, before anything has finished, must wait
    for those conversions - both give the result of a call made after everything has drained."""
    import torch
    B, S, d, ffn, H = 4, 256, 1024, 1024, 8
    f = lambda *s, sc=0.03: to_dev((sc * rng.standard_normal(s)).astype(np.float32), gpu)
    x = to_dev(rng.standard_normal((B, S, d)).astype(np.float32), gpu)
    lib = pkg.ops()
    for trial in range(3):
        W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]   # new arrays: the cache has not seen them
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        torch.cuda.synchronize()
        lib.mgpuLLMOpsCacheWeights(1)
        try:
            a = pkg.decoding_context_layer(x, *W, heads=H, stream=s1)
            b = pkg.decoding_context_layer(x, *W, heads=H, stream=s2)
            torch.cuda.synchronize()
            settled = pkg.decoding_context_layer(x, *W, heads=H)
            torch.cuda.synchronize()
        finally:
            lib.mgpuLLMOpsCacheWeights(0)
        assert torch.equal(a, settled) and torch.equal(b, settled), trial
    assert lib.mgpuOpsTakeLastError() is None


def test_bert_encoder_layer_weight_cache(pkg, gpu, oracle):
    """With mgpuLLMOpsCacheWeights(1) the BERT layer hands the GEMMs the committed table marks (QKV and FFN2 at
    configs[4]) a transposed copy of their weight, kept by the cache: same layer against the oracle, the same
    bits on the second call, and an odd shape (nothing in the table, library everywhere) as well."""
    import torch
    rng = np.random.Generator(np.random.PCG64(20246))
    lib = pkg.ops()
    for B, S, d, ffn, H in ((32, 128, 768, 3072, 12), (3, 50, 192, 200, 3)):
        h16 = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float16)
        gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
        x = rng.standard_normal((B, S, d)).astype(np.float16)
        P = [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
             h16(d), gam(), h16(d)]
        dev = [to_dev(p, gpu) for p in P]
        ref = oracle.bert_layer_f16(x, *P, heads=H)
        lib.mgpuLLMOpsCacheWeights(1)
        try:
            first = pkg.bert_encoder_layer(to_dev(x, gpu), *dev, heads=H).clone()
            again = pkg.bert_encoder_layer(to_dev(x, gpu), *dev, heads=H).clone()
        finally:
            lib.mgpuLLMOpsCacheWeights(0)
        assert torch.equal(first, again)
        err = np.abs(first.cpu().numpy().astype(np.float32) - ref)
        assert np.all(err <= layer_tol(ref)), err.max()
        assert err.mean() <= 5e-4
    assert lib.mgpuOpsTakeLastError() is None


@pytest.mark.parametrize("causal,relu,d,H", [(True, True, 512, 8), (False, False, 512, 8), (True, True, 1024, 8),
                                             (True, False, 512, 2)])
def test_decoding_context_layer(pkg, gpu, oracle, rng, causal, relu, d, H):
    """(1024, 8): the reference's own head geometry, 8 heads of 128; (512, 2): heads of 256, the widest of the
    reference's attention kernel list."""
    B, S, ffn = 4, 128, 2048
    f = lambda *s, sc=0.03: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    got = pkg.decoding_context_layer(to_dev(x, gpu), *[to_dev(w, gpu) for w in W], heads=H, causal=causal,
                                     relu=relu).cpu().numpy()
    ref = oracle.decoding_context_layer(x, *W, heads=H, causal=causal,
                                        act=oracle.ACT_RELU if relu else oracle.ACT_GELU)
    err = np.abs(got - ref)
    assert np.all(err <= layer_tol(ref)), err.max()
    # output is fp16-representable fp32, like the reference's final cast
    assert np.array_equal(got, got.astype(np.float16).astype(np.float32))


def test_decoding_context_layer_weight_cache(pkg, gpu, oracle, rng):
    """mgpuLLMOpsCacheWeights(1): the fp32 weights are cast once, when first seen (the matrices into a transposed
    fp16 copy that a different library kernel multiplies, so the result is checked against the oracle, not against
    the bits of the per-call path), and later calls reuse the copies; switching the cache off and on again drops
    them, so weights changed in place in between are picked up."""
    import torch
    B, S, d, ffn, H = 2, 128, 512, 1024, 8
    f = lambda *s, sc=0.03: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    Wh = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    xd, W = to_dev(x, gpu), [to_dev(w, gpu) for w in Wh]
    lib = pkg.ops()

    def close(got, weights):
        ref = oracle.decoding_context_layer(x, *weights, heads=H)
        err = np.abs(got.cpu().numpy() - ref)
        return bool(np.all(err <= layer_tol(ref))) and err.mean() <= 5e-4

    plain = pkg.decoding_context_layer(xd, *W, heads=H).clone()
    lib.mgpuLLMOpsCacheWeights(1)
    try:
        first = pkg.decoding_context_layer(xd, *W, heads=H).clone()     # fills the cache
        again = pkg.decoding_context_layer(xd, *W, heads=H).clone()     # served from it
        assert close(first, Wh) and torch.equal(again, first)
        assert (first - plain).abs().max().item() <= 2e-2               # another kernel's rounding, no more
        W[1].mul_(0.5)                                                  # in place: the cache does not see it
        stale = pkg.decoding_context_layer(xd, *W, heads=H).clone()
        assert torch.equal(stale, first)
        lib.mgpuLLMOpsCacheWeights(0)
        lib.mgpuLLMOpsCacheWeights(1)
        fresh = pkg.decoding_context_layer(xd, *W, heads=H).clone()
    finally:
        lib.mgpuLLMOpsCacheWeights(0)
    Wh[1] = Wh[1] * np.float32(0.5)
    assert close(fresh, Wh) and not close(fresh, [w if i != 1 else w * np.float32(2) for i, w in enumerate(Wh)])
    assert close(pkg.decoding_context_layer(xd, *W, heads=H), Wh)       # per-call casts again
    assert lib.mgpuOpsTakeLastError() is None


@pytest.mark.parametrize("causal,relu,d,H", [(True, True, 512, 8), (False, False, 768, 12)])
def test_decoding_context_layer_post_ln(pkg, gpu, oracle, rng, causal, relu, d, H):
    """norm_first = false (Ops.h:43-48 declares the flag; the reference's bodies never read it): the post-LN
    ordering, h = LN(x + proj(attention(x))), out = LN(h + ffn(h)).  The pre-LN result of the same
    operands must differ, so a flag that is dropped on the way fails here."""
    B, S, ffn = 4, 128, 2048
    f = lambda *s, sc=0.03: (sc * rng.standard_normal(s)).astype(np.float32)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    dev = [to_dev(w, gpu) for w in W]
    got = pkg.decoding_context_layer(to_dev(x, gpu), *dev, heads=H, causal=causal, relu=relu,
                                     norm_first=False).cpu().numpy()
    act = oracle.ACT_RELU if relu else oracle.ACT_GELU
    ref = oracle.decoding_context_layer(x, *W, heads=H, causal=causal, act=act, norm_first=False)
    err = np.abs(got - ref)
    assert np.all(err <= layer_tol(ref)), err.max()
    assert err.mean() <= 5e-4
    assert np.array_equal(got, got.astype(np.float16).astype(np.float32))
    pre = pkg.decoding_context_layer(to_dev(x, gpu), *dev, heads=H, causal=causal, relu=relu).cpu().numpy()
    assert np.abs(pre - got).max() > 0.1
