"""Pins oracle_fmha (oracle/oracle.c) against torch's CPU attention in fp64,
brute-force Python loops on tiny cases, and identities of softmax attention.
The reference's own arithmetic for this op sits in opaque cubins, so parity
with ITS rounding sequence stays unpinned; what is pinned is the function
softmax(scale QK^T + mask) V on the packed [B,S,3,H,D] layout.  CPU only."""
import math

import numpy as np
import torch


def _torch_ref(qkv, lens=None, causal=False, scale=None):
    B, S, _, H, D = qkv.shape
    t = torch.from_numpy(qkv.astype(np.float64))
    q, k, v = [t[:, :, i].permute(0, 2, 1, 3) for i in range(3)]  # [B,H,S,D]
    mask = torch.ones(B, 1, S, S, dtype=torch.bool)
    if lens is not None:
        for b, l in enumerate(lens):
            mask[b, :, :, l:] = False
    if causal:
        mask &= torch.tril(torch.ones(S, S, dtype=torch.bool))
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=scale)
    return o.permute(0, 2, 1, 3).reshape(B, S, H * D).numpy()


def test_fmha_against_torch_sdpa(oracle, rng):
    for (B, S, H, lens, causal) in [(2, 128, 3, None, False), (2, 77, 2, [77, 30], False),
                                    (1, 64, 2, None, True), (2, 96, 1, [50, 96], True)]:
        qkv = (rng.standard_normal((B, S, 3, H, 64)) / 8).astype(np.float16)
        got = oracle.fmha(qkv, lens, causal=causal)
        ref = _torch_ref(qkv, lens, causal)
        assert np.abs(got - ref).max() < 2e-7, (B, S, H, lens, causal)


def test_fmha_brute_force_tiny(oracle, rng):
    """Pure-python loops over the packed layout: catches a wrong stride, a
    transposed operand or a head/which mix-up in the indexing."""
    B, S, H, D = 2, 5, 3, 8
    qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float16)
    lens = [5, 3]
    scale = 0.3
    got = oracle.fmha(qkv, lens, scale=scale)
    flat = qkv.astype(np.float64).reshape(-1)

    def at(b, s, w, h, d):
        return flat[(((b * S + s) * 3 + w) * H + h) * D + d]

    for b in range(B):
        for h in range(H):
            for i in range(S):
                sc = [scale * sum(at(b, i, 0, h, d) * at(b, j, 1, h, d) for d in range(D)) for j in range(lens[b])]
                mx = max(sc)
                p = [math.exp(s - mx) for s in sc]
                den = sum(p)
                for d in range(D):
                    o = sum(p[j] * at(b, j, 2, h, d) for j in range(lens[b])) / den
                    assert abs(got[b, i, h * D + d] - o) < 1e-6


def test_fmha_identities(oracle, rng):
    B, S, H, D = 2, 48, 2, 64
    qkv = (rng.standard_normal((B, S, 3, H, D)) / 4).astype(np.float16)
    lens = np.array([48, 20], np.int32)
    # V constant per head -> output is that constant (rows of P sum to one)
    c = qkv.copy()
    c[:, :, 2] = np.float16(0.375)
    assert np.allclose(oracle.fmha(c, lens), 0.375, atol=1e-7)
    # Q = 0 -> uniform weights -> mean of the valid V rows
    z = qkv.copy()
    z[:, :, 0] = 0
    out = oracle.fmha(z, lens)
    for b in range(B):
        mean_v = z[b, : lens[b], 2].astype(np.float64).mean(0).reshape(-1)
        assert np.allclose(out[b], mean_v[None, :], atol=1e-6)
    # permuting the valid keys (K and V rows together) leaves O unchanged
    perm = rng.permutation(20)
    p = qkv.copy()
    p[1, :20, 1:] = qkv[1, perm, 1:]
    assert np.allclose(oracle.fmha(p, lens)[1], oracle.fmha(qkv, lens)[1], atol=1e-6)
    # masked keys do not matter at all
    g = qkv.copy()
    g[1, 20:, 1:] = np.float16(9.0)
    assert np.array_equal(oracle.fmha(g, lens), oracle.fmha(qkv, lens))
    # S = 1 (or causal row 0): O = V
    one = qkv[:, :1]
    assert np.allclose(oracle.fmha(one), one[:, :, 2].astype(np.float32).reshape(B, 1, H * D), atol=1e-7)
    assert np.allclose(oracle.fmha(qkv, causal=True)[:, 0], qkv[:, 0, 2].astype(np.float32).reshape(B, H * D), atol=1e-7)
    # scale enters the logits: scale -> 0 gives the plain mean
    out = oracle.fmha(qkv, scale=1e-12)
    assert np.allclose(out[0], qkv[0, :, 2].astype(np.float64).mean(0).reshape(-1)[None, :], atol=1e-6)


def test_fmha_edge_lengths(oracle, rng):
    qkv = (rng.standard_normal((3, 16, 3, 1, 64)) / 8).astype(np.float16)
    out = oracle.fmha(qkv, np.array([0, 1, 16], np.int32))
    assert np.all(out[0] == 0)  # no admissible key -> zeros
    assert np.allclose(out[1], qkv[1, 0, 2].astype(np.float32).reshape(-1)[None, :], atol=1e-7)
    # lengths beyond S clamp to S
    assert np.array_equal(oracle.fmha(qkv, np.array([99, 99, 99], np.int32)), oracle.fmha(qkv))


def test_fmha_bf16_inputs(oracle, rng):
    f = (rng.standard_normal((1, 32, 3, 2, 64)) / 8).astype(np.float32)
    bits = oracle.float_to_bf16(f)
    got = oracle.fmha(bits, bf16=True)
    ref = _torch_ref(oracle.bf16_to_float(bits))
    assert np.abs(got - ref).max() < 2e-7
