"""Parity of the HIP fused multi-head attention (C ABI mgpuFusedMHAF16 / BF16)
with the oracle, on unit-variance inputs (logits ~ N(0, 1) at scale 1/8, outputs
O(0.1 .. 1)): |error| <= 2e-3 * max(1, |ref|) elementwise on fp16 outputs
against the fp64 CPU result, i.e. max abs error <= 2e-3 wherever the output is
below 1 and one fp16 spacing above that (bf16: 8e-3, its spacing below 1 being
2^-8)."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu

TOL_F16 = 2e-3
TOL_BF16 = 8e-3


def excess(got, ref, tol):
    """Largest |got - ref| in units of the allowed bound tol * max(1, |ref|)."""
    return float((np.abs(got - ref) / (tol * np.maximum(1.0, np.abs(ref)))).max()) if ref.size else 0.0


def run(pkg, gpu, qkv, lens=None, causal=False, scale=None):
    tl = to_dev(np.asarray(lens, np.int32), gpu) if lens is not None else None
    return pkg.fused_mha(to_dev(qkv, gpu), tl, scale=scale, causal=causal).cpu().numpy().astype(np.float32)


def make_qkv(rng, B, S, H, std=1.0, D=64):
    # unit variance: logits ~ N(0, 1) at scale 1/8, outputs O(0.1 .. 1) - an error in
    # the softmax weights or a V tile paired with the wrong P is far above tolerance
    return (rng.standard_normal((B, S, 3, H, D)) * std).astype(np.float16)


def test_fmha_config2_b32_s128_h12(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20242))
    qkv = make_qkv(rng, 32, 128, 12, std=1.0 / 8)  # the configuration's own draw
    got = run(pkg, gpu, qkv)
    assert np.abs(got - oracle.fmha(qkv)).max() <= TOL_F16
    qkv = make_qkv(rng, 32, 128, 12)
    got = run(pkg, gpu, qkv)
    assert excess(got, oracle.fmha(qkv), TOL_F16) <= 1.0


def test_fmha_config3_b8_s512_h16_key_padding(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20243))
    lens = rng.integers(256, 513, 8).astype(np.int32)
    qkv = make_qkv(rng, 8, 512, 16, std=1.0 / 8)  # the configuration's own draw
    got = run(pkg, gpu, qkv, lens)
    assert np.abs(got - oracle.fmha(qkv, lens)).max() <= TOL_F16
    qkv = make_qkv(rng, 8, 512, 16)
    got = run(pkg, gpu, qkv, lens)
    assert excess(got, oracle.fmha(qkv, lens), TOL_F16) <= 1.0


def test_fmha_roofline_shape_b32_s512_h12(pkg, gpu, oracle):
    rng = np.random.Generator(np.random.PCG64(20244))
    qkv = make_qkv(rng, 32, 512, 12)
    got = run(pkg, gpu, qkv)
    assert excess(got, oracle.fmha(qkv), TOL_F16) <= 1.0


# ragged S (partial query blocks and partial key tiles), S below one tile,
# lengths of 0 / 1 / exactly on and one past a tile boundary
@pytest.mark.parametrize("B,S,H,lens", [
    (1, 1, 1, None), (2, 5, 2, None), (1, 63, 1, None), (1, 64, 2, None), (1, 65, 1, None),
    (2, 127, 3, None), (1, 129, 2, None), (2, 200, 3, [1, 150]), (3, 192, 2, [64, 65, 128]),
    (2, 300, 1, [300, 299]), (4, 96, 2, [0, 1, 2, 96]), (1, 1000, 1, [777]), (2, 128, 4, [500, -3]),
])
def test_fmha_ragged_and_masked(pkg, gpu, oracle, rng, B, S, H, lens):
    qkv = make_qkv(rng, B, S, H)
    got = run(pkg, gpu, qkv, lens)
    ref = oracle.fmha(qkv, lens)
    assert excess(got, ref, TOL_F16) <= 1.0
    if lens is not None:
        for b, l in enumerate(lens):
            if l <= 0:
                assert np.all(got[b] == 0)  # no admissible key -> zeros


@pytest.mark.parametrize("B,S,H,lens", [(2, 128, 2, None), (1, 257, 2, None), (2, 512, 1, [512, 100]),
                                        (1, 70, 3, [33])])
def test_fmha_causal(pkg, gpu, oracle, rng, B, S, H, lens):
    qkv = make_qkv(rng, B, S, H)
    got = run(pkg, gpu, qkv, lens, causal=True)
    assert excess(got, oracle.fmha(qkv, lens, causal=True), TOL_F16) <= 1.0


def causal_blocks_are_paired(B, S, H, cus):
    """The launcher's rule: exactly four query blocks per (batch, head) and a halved grid of two work items per CU."""
    return (S + 127) // 128 == 4 and B * H * 2 >= 2 * cus


@pytest.mark.parametrize("D,B,S,H,ragged,dtype", [
    (64, 32, 512, 12, False, "f16"),   # four query blocks per (batch, head): pairs (3, 0) and (2, 1)
    (64, 16, 500, 16, True, "f16"),    # the last block twelve rows short; ragged key counts
    (128, 32, 512, 8, False, "f16"),   # the 128-wide geometry, exactly two work items per CU
    (128, 16, 450, 16, True, "bf16"),  # its last block two rows long
    (40, 32, 512, 12, True, "f16"),    # a head size padded into the 64-wide geometry
])
def test_fmha_causal_paired_query_blocks(pkg, gpu, oracle, D, B, S, H, ragged, dtype):
    """With four query blocks per (batch, head) on grids that leave every CU two work items afterwards, the
    causal kernel gives query block i and block 3 - i to one work item, which runs them one after the
    other through the same LDS ring; the small problems of the other causal tests never get there."""
    import torch
    assert causal_blocks_are_paired(B, S, H, torch.cuda.get_device_properties(gpu).multi_processor_count)
    rng = np.random.Generator(np.random.PCG64(D * 1000 + S))
    tq = torch.from_numpy(rng.standard_normal((B, S, 3, H, D)).astype(np.float32)).to(gpu)
    tq = tq.to(torch.float16 if dtype == "f16" else torch.bfloat16)
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
    lens = None
    if ragged:
        lens = rng.integers(0, S + 1, B).astype(np.int32)
        lens[0], lens[1] = S, 1
    got = pkg.fused_mha(tq, to_dev(lens, gpu) if ragged else None, causal=True).float().cpu().numpy()
    ref = oracle.fmha(bits.view(np.float16) if dtype == "f16" else bits, lens, causal=True, bf16=dtype == "bf16")
    assert excess(got, ref, TOL_F16 if dtype == "f16" else TOL_BF16) <= 1.0


@pytest.mark.parametrize("D,B,S,H,ragged,packed", [
    (64, 8, 640, 8, True, False),     # five query blocks per (batch, head), 320 blocks: 40 per XCD, longest first
    (128, 8, 512, 16, False, False),  # the reference layer's attention at (8,512,2048): 512 blocks, two per CU
    (64, 16, 640, 16, True, False),   # 1280 blocks: several rounds; ragged key counts
    (128, 16, 384, 16, True, False),  # three query blocks, 128-wide heads
    (64, 16, 300, 8, False, True),    # packed rows of unequal length under the same order
    (64, 5, 640, 12, False, False),   # 300 blocks, not a multiple of 8: longest first over the whole grid
    (64, 4, 768, 11, False, False),   # 264 blocks, 33 per XCD, not whole (batch, head)s: the same
])
def test_fmha_causal_longest_block_first(pkg, gpu, oracle, D, B, S, H, ragged, packed):
    """Causal grids with more blocks than CUs that are not paired: the launcher has the kernel hand out each XCD's
    query blocks longest first (another map from block id to (batch, head, query block)); every row of every
    block must still come out."""
    import torch
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    assert cus < B * H * ((S + 127) // 128) and not causal_blocks_are_paired(B, S, H, cus)
    rng = np.random.Generator(np.random.PCG64(D * 977 + S + B))
    if packed:
        lens = rng.integers(1, S + 1, B)
        lens[:3] = [S, 1, 129]
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        tq = torch.from_numpy(rng.standard_normal((int(cu[-1]), 3, H, D)).astype(np.float32)).to(gpu).half()
        got = pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), S, causal=True).float().cpu().numpy()
        bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
        for b in range(B):
            ref = oracle.fmha(bits[cu[b]:cu[b + 1]][None].view(np.float16), causal=True)[0]
            assert excess(got[cu[b]:cu[b + 1]], ref, TOL_F16) <= 1.0, f"sequence {b} of {lens[b]} rows"
        return
    qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float16)
    lens = None
    if ragged:
        lens = rng.integers(0, S + 1, B).astype(np.int32)
        lens[0], lens[1] = S, 1
    got = run(pkg, gpu, qkv, lens, causal=True)
    assert excess(got, oracle.fmha(qkv, lens, causal=True), TOL_F16) <= 1.0


def test_fmha_seeded_sweep_over_the_block_orders(pkg, gpu, oracle):
    """A seeded draw of shapes, masks and length forms: whatever order the launcher hands the blocks out in (index
    order, pairs, longest first, (batch, head)s dealt over the XCDs, packed rows), every output row is the
    attention of its own query over its own keys."""
    import random
    import torch
    rnd = random.Random(20250)
    cases = 0
    while cases < 14:
        D = rnd.choice([64, 64, 128, 40])
        H, B = rnd.choice([1, 3, 4, 8, 12, 16]), rnd.choice([1, 2, 5, 8, 16])
        S = rnd.choice([64, 200, 256, 384, 512, 640])
        if B * H * S * S * D > 1.2e9:
            continue
        causal, mode = rnd.random() < 0.5, rnd.choice(["dense", "seqlens", "cu"])
        rng = np.random.Generator(np.random.PCG64(1000 + cases))
        cases += 1
        if mode == "cu":
            lens = np.array([rnd.randint(0, S) for _ in range(B)])
            lens[0] = S
            cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            qkv = rng.standard_normal((int(cu[-1]), 3, H, D)).astype(np.float16)
            got = pkg.fused_mha_cu_seqlens(to_dev(qkv, gpu), to_dev(cu, gpu), S, causal=causal).float().cpu().numpy()
            for b in range(B):
                if lens[b]:
                    ref = oracle.fmha(qkv[cu[b]:cu[b + 1]][None], causal=causal)[0]
                    assert excess(got[cu[b]:cu[b + 1]], ref, TOL_F16) <= 1.0, (D, B, S, H, causal, mode, b)
        else:
            qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float16)
            lens = np.array([rnd.randint(0, S) for _ in range(B)], np.int32) if mode == "seqlens" else None
            got = run(pkg, gpu, qkv, lens, causal=causal)
            assert excess(got, oracle.fmha(qkv, lens, causal=causal), TOL_F16) <= 1.0, (D, B, S, H, causal, mode)


def test_fmha_causal_paired_query_blocks_over_packed_rows(pkg, gpu, oracle):
    """The same pairing with the sequences given as prefix sums over packed rows: a pair's late block may lie
    wholly beyond a short sequence while its early block does not."""
    import torch
    B, S, H, D = 40, 512, 8, 64
    rng = np.random.Generator(np.random.PCG64(4051))
    lens = rng.integers(0, S + 1, B)
    lens[:6] = [S, 0, 1, 128, 129, 385]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tq = torch.from_numpy(rng.standard_normal((int(cu[-1]), 3, H, D)).astype(np.float32)).to(gpu).half()
    guard = torch.full((int(cu[-1]) + 64, H * D), 7.0, device=gpu, dtype=torch.float16)
    pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), S, causal=True, out=guard[:int(cu[-1])])
    assert (guard[int(cu[-1]):] == 7.0).all()  # nothing written past the last row
    got = guard[:int(cu[-1])].float().cpu().numpy()
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
    for b, n in enumerate(lens):
        if n:
            ref = oracle.fmha(bits[cu[b]:cu[b + 1]][None].view(np.float16), causal=True)[0]
            assert excess(got[cu[b]:cu[b + 1]], ref, TOL_F16) <= 1.0, f"sequence {b} of {n} rows"


def test_fmha_large_logits_and_other_scales(pkg, gpu, oracle, rng):
    """Peaked softmax rows: the kernel produces P against a stale reference
    maximum and repairs overflow after the fact, so rows whose scores keep
    growing from tile to tile (scale 1.0: logits ~ N(0, 64), up to +-40) take
    the repair path over and over.  The scale is a free fp32 parameter of the
    entry point and is applied in fp32, so the bound does not move with it."""
    qkv = make_qkv(rng, 2, 256, 2)
    for scale in (0.01, 0.125, 0.5, 1.0):
        got = run(pkg, gpu, qkv, scale=scale)
        assert excess(got, oracle.fmha(qkv, scale=scale), TOL_F16) <= 1.0, scale
    for std in (1.6, 3.0):  # |logits| up to ~12 and ~40 at the default scale, outputs up to ~13
        qkv = make_qkv(rng, 2, 320, 2, std=std)
        assert excess(run(pkg, gpu, qkv), oracle.fmha(qkv), TOL_F16) <= 1.0, std
    # a row maximum that rises by far more than fp16's range from one tile to the next
    qkv = make_qkv(rng, 1, 256, 1)
    qkv[0, :, 1, 0, :] *= np.linspace(0.05, 6.0, 256, dtype=np.float16)[:, None]
    assert excess(run(pkg, gpu, qkv, scale=1.0), oracle.fmha(qkv, scale=1.0), TOL_F16) <= 1.0


@pytest.mark.parametrize("D", [64, 128])
def test_fmha_logits_far_from_zero(pkg, gpu, oracle, rng, D):
    """The kernel's first softmax reference is 0.  Logits that all sit far below
    it (every p underflows on the first pass) or far above it (every p
    overflows) must be caught on the first tile; a common offset of all of a
    row's logits does not change the softmax."""
    B, S, H = 1, 200, 2
    qkv = make_qkv(rng, B, S, H, std=0.5, D=D)
    u = np.zeros(D, np.float16)
    u[:8] = 4.0
    for sign in (-1.0, 1.0):  # q.k moves by -+128: logits near -+16 (D = 64) or -+11 (D = 128) plus noise
        shifted = qkv.copy()
        shifted[:, :, 0, 0, :] += np.float16(sign) * u   # queries of head 0
        shifted[:, :, 1, 0, :] += u                      # keys of head 0
        ref = oracle.fmha(shifted)
        got = run(pkg, gpu, shifted)
        assert np.isfinite(got).all() and excess(got, ref, TOL_F16) <= 1.0, sign
    # first tile far below the reference, later keys far above the first tile
    ramp = qkv.copy()
    ramp[:, :, 0, :, :] = 0
    ramp[:, :, 0, :, 0] = 8.0
    ramp[:, :, 1, :, 0] = np.linspace(-60.0, 60.0, S, dtype=np.float16)[None, :, None]
    for causal in (False, True):
        ref = oracle.fmha(ramp, causal=causal)
        got = run(pkg, gpu, ramp, causal=causal)
        assert np.isfinite(got).all() and excess(got, ref, TOL_F16) <= 1.0, causal


@pytest.mark.parametrize("B,S,H,lens,causal", [
    (2, 128, 8, None, False), (1, 1, 1, None, False), (2, 31, 2, None, False), (1, 32, 1, None, True),
    (2, 33, 2, [33, 7], False), (1, 257, 3, None, True), (2, 512, 2, [512, 300], False), (3, 100, 2, [0, 1, 100], True),
    (1, 1000, 1, [777], False),
])
def test_fmha_head_dim_128(pkg, gpu, oracle, rng, B, S, H, lens, causal):
    """head_dim 128 (the reference's layer runs 8 heads of 128, LLM.cu:79-81 with
    qkvToContext.cu:62-75): key tiles of 32, default scale 1/sqrt(128)."""
    qkv = make_qkv(rng, B, S, H, D=128)
    got = run(pkg, gpu, qkv, lens, causal=causal)
    ref = oracle.fmha(qkv, lens, causal=causal)
    assert got.shape == (B, S, H * 128)
    assert excess(got, ref, TOL_F16) <= 1.0
    dirty = qkv.copy()
    if lens is not None:  # padding may hold anything
        for b, l in enumerate(lens):
            dirty[b, max(l, 0):, 1:] = np.float16(np.nan)
        got = run(pkg, gpu, dirty, lens, causal=causal)
        assert np.isfinite(got).all() and excess(got, ref, TOL_F16) <= 1.0


def test_fmha_head_dim_128_bf16_and_peaked(pkg, gpu, oracle, rng):
    import torch
    f = rng.standard_normal((2, 200, 3, 2, 128)).astype(np.float32)
    t = torch.from_numpy(f).to(gpu).to(torch.bfloat16)
    got = pkg.fused_mha(t).float().cpu().numpy()
    bits = t.view(torch.int16).cpu().numpy().view(np.uint16)
    assert excess(got, oracle.fmha(bits, bf16=True), TOL_BF16) <= 1.0
    qkv = make_qkv(rng, 1, 320, 2, D=128)
    for scale in (1.0 / np.sqrt(128), 0.5):  # 0.5: logits ~ N(0, 32), repeated overflow repair
        assert excess(run(pkg, gpu, qkv, scale=scale), oracle.fmha(qkv, scale=scale), TOL_F16) <= 1.0, scale


def test_fmha_padding_garbage_is_ignored(pkg, gpu, oracle, rng):
    """Keys past the valid length may hold anything, NaN and Inf included."""
    qkv = make_qkv(rng, 2, 160, 2)
    lens = [100, 37]
    ref = oracle.fmha(qkv, lens)
    dirty = qkv.copy()
    for b, l in enumerate(lens):
        dirty[b, l:, 1:] = np.float16(np.nan)
        dirty[b, l::2, 1:] = np.float16(np.inf)
    got = run(pkg, gpu, dirty, lens)
    assert np.isfinite(got).all() and excess(got, ref, TOL_F16) <= 1.0


def test_fmha_identities_at_full_size(pkg, gpu):
    """Size-independent properties at the roofline shape (b32 s512 h12):
    constant V gives that constant, Q = 0 gives the mean of V, permuting the
    keys (K and V rows together) changes nothing beyond rounding."""
    import torch
    g = torch.Generator(device=gpu)
    g.manual_seed(11)
    B, S, H = 32, 512, 12
    qkv = torch.randn((B, S, 3, H, 64), device=gpu, generator=g).half()
    base = pkg.fused_mha(qkv).float()
    c = qkv.clone()
    c[:, :, 2] = 0.375
    assert (pkg.fused_mha(c).float() - 0.375).abs().max().item() <= 1e-3
    z = qkv.clone()
    z[:, :, 0] = 0
    mean_v = z[:, :, 2].float().mean(1).reshape(B, 1, H * 64)
    assert (pkg.fused_mha(z).float() - mean_v).abs().max().item() <= 1e-3
    perm = torch.randperm(S, device=gpu, generator=g)
    p = qkv.clone()
    p[:, :, 1:] = qkv[:, perm, 1:]
    assert (pkg.fused_mha(p).float() - base).abs().max().item() <= 2e-3
    assert torch.equal(pkg.fused_mha(qkv), pkg.fused_mha(qkv))  # deterministic


@pytest.mark.parametrize("B,S,H,ragged,dtype", [(8, 2048, 8, False, "f16"), (4, 2304, 16, True, "f16"),
                                                 (8, 2048, 8, True, "bf16")])
def test_fmha_long_sequences_with_64_queries_per_wavefront(pkg, gpu, oracle, B, S, H, ragged, dtype):
    """From S = 2048 on, with enough (batch, head) pairs to give every CU two blocks of 256 queries, the
    unmasked / key-padded head_dim-64 problem runs with 64 queries per wavefront (another instantiation of
    the kernel): against the oracle with unit-variance operands, partial last query block (2304 = 9 x 256)
    and ragged key counts included, and against the 32-query kernel, which the causal flag selects on a
    problem whose mask hides nothing (key counts of 1: one admissible key per row either way)."""
    import torch
    rng = np.random.Generator(np.random.PCG64(S + H))
    qkv = rng.standard_normal((B, S, 3, H, 64)).astype(np.float32)
    lens = rng.integers(1, S + 1, B).astype(np.int32) if ragged else None
    if ragged:
        lens[0] = S
    tq = torch.from_numpy(qkv).to(gpu).to(torch.float16 if dtype == "f16" else torch.bfloat16)
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
    tl = to_dev(lens, gpu) if ragged else None
    got = pkg.fused_mha(tq, tl).float().cpu().numpy()
    ref = oracle.fmha(bits.view(np.float16) if dtype == "f16" else bits, lens, bf16=dtype == "bf16")
    assert excess(got, ref, TOL_F16 if dtype == "f16" else TOL_BF16) <= 1.0
    one = to_dev(np.ones(B, np.int32), gpu)
    a = pkg.fused_mha(tq, one).float()
    b = pkg.fused_mha(tq, one, causal=True).float()
    assert (a - b).abs().max().item() <= 1e-6


def test_fmha_long_packed_rows_with_64_queries_per_wavefront(pkg, gpu, oracle):
    """The 64-query instantiation behind the prefix-sum entry point: sequences of up to 2048 packed rows, among them
    an empty one, one of a single row, and lengths either side of the 256-query block size."""
    import torch
    B, S, H = 8, 2048, 8
    rng = np.random.Generator(np.random.PCG64(77))
    lens = np.array([S, 0, 1, 255, 256, 257, 1300, 2047])
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    total = int(cu[-1])
    tq = torch.from_numpy(rng.standard_normal((total, 3, H, 64)).astype(np.float32)).to(gpu).half()
    guard = torch.full((total + 64, H * 64), 7.0, device=gpu, dtype=torch.float16)
    pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), S, out=guard[:total])
    assert (guard[total:] == 7.0).all()
    got = guard[:total].float().cpu().numpy()
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
    for b, n in enumerate(lens):
        if n:
            ref = oracle.fmha(bits[cu[b]:cu[b + 1]][None].view(np.float16))[0]
            assert excess(got[cu[b]:cu[b + 1]], ref, TOL_F16) <= 1.0, f"sequence {b} of {n} rows"


def test_fmha_seeded_shape_sweep(pkg, gpu, oracle):
    """Forty problems drawn from a fixed seed over everything the entry points take: head sizes
    8..256 (all three tile geometries and the sizes padded into them), S from 1 to a few tiles past
    the block sizes, key counts with zeros and full lengths, causal or not, fp16 or bf16, padded
    layout or packed rows behind prefix sums - each against the oracle."""
    import torch
    rng = np.random.Generator(np.random.PCG64(20260))
    for case in range(40):
        D = int(rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 80, 96, 104, 128, 136, 144, 160, 192, 248, 256]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        S = int(rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 191, 200, 256, 257, 300, 385, 512, 640]))
        causal = bool(rng.integers(0, 2))
        bf16 = bool(rng.integers(0, 4) == 0)
        mode = int(rng.integers(0, 3))  # 0: no lengths, 1: key counts, 2: packed rows with prefix sums
        dt = torch.bfloat16 if bf16 else torch.float16
        tol = TOL_BF16 if bf16 else TOL_F16
        what = f"case {case}: D={D} B={B} H={H} S={S} causal={causal} bf16={bf16} mode={mode}"
        if mode < 2:
            lens = None
            if mode == 1:
                lens = rng.integers(0, S + 1, B).astype(np.int32)
                lens[rng.integers(0, B)] = S
            tq = torch.from_numpy(rng.standard_normal((B, S, 3, H, D)).astype(np.float32)).to(gpu).to(dt)
            bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
            got = pkg.fused_mha(tq, to_dev(lens, gpu) if lens is not None else None, causal=causal).float().cpu().numpy()
            ref = oracle.fmha(bits if bf16 else bits.view(np.float16), lens, causal=causal, bf16=bf16)
            assert excess(got, ref, tol) <= 1.0, what
        else:
            lens = rng.integers(0, S + 1, B)
            lens[rng.integers(0, B)] = S
            cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            tq = torch.from_numpy(rng.standard_normal((int(cu[-1]), 3, H, D)).astype(np.float32)).to(gpu).to(dt)
            got = pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), S, causal=causal).float().cpu().numpy()
            bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
            for b, n in enumerate(lens):
                if n:
                    rows = bits[cu[b]:cu[b + 1]][None]
                    ref = oracle.fmha(rows if bf16 else rows.view(np.float16), causal=causal, bf16=bf16)[0]
                    assert excess(got[cu[b]:cu[b + 1]], ref, tol) <= 1.0, what + f" sequence {b}"


def test_fmha_bf16(pkg, gpu, oracle, rng):
    import torch
    for (B, S, H, lens, causal) in [(2, 128, 2, None, False), (2, 200, 3, [200, 77], False), (1, 130, 1, None, True)]:
        f = rng.standard_normal((B, S, 3, H, 64)).astype(np.float32)
        t = torch.from_numpy(f).to(gpu).to(torch.bfloat16)
        tl = to_dev(np.asarray(lens, np.int32), gpu) if lens is not None else None
        got = pkg.fused_mha(t, tl, causal=causal).float().cpu().numpy()
        bits = t.view(torch.int16).cpu().numpy().view(np.uint16)
        ref = oracle.fmha(bits, lens, causal=causal, bf16=True)
        assert excess(got, ref, TOL_BF16) <= 1.0


@pytest.mark.parametrize("lens,max_s,causal,D,dtype", [
    ([128, 128, 128], 128, False, 64, "f16"),          # the dense call written as prefix sums
    ([5, 0, 300, 64, 1, 129], 300, False, 64, "f16"),  # ragged, an empty sequence, tile boundaries
    ([200, 77, 512], 512, True, 64, "f16"),            # causal over packed rows
    ([33, 250], 256, False, 128, "f16"),
    ([100, 260], 260, True, 64, "bf16"),
])
def test_fmha_cu_seqlens_packed_rows(pkg, gpu, oracle, rng, lens, max_s, causal, D, dtype):
    """The reference's own description of the batch (fused_multihead_attention_v2.h:63-64):
    b + 1 prefix sums over token rows packed back to back.  Each sequence must come out
    as the dense attention of that sequence alone, and no row of a neighbour is touched."""
    import torch
    H = 3
    total = int(np.sum(lens))
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qkv = rng.standard_normal((total, 3, H, D)).astype(np.float32)
    tq = torch.from_numpy(qkv).to(gpu).to(torch.float16 if dtype == "f16" else torch.bfloat16)
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)  # the rounded values, as bit patterns
    out = torch.full((total + 1, H * D), 7.0, dtype=tq.dtype, device=gpu)  # one guard row behind the batch
    pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), max_s, causal=causal, out=out[:total])
    got = out.float().cpu().numpy()
    assert np.all(got[total] == 7.0)
    tol = TOL_F16 if dtype == "f16" else TOL_BF16
    for b, n in enumerate(lens):
        if n == 0:
            continue
        seq = bits[cu[b]:cu[b + 1]][None]  # [1, n, 3, H, D]
        ref = oracle.fmha(seq.view(np.float16) if dtype == "f16" else seq, None, causal=causal, bf16=dtype == "bf16")[0]
        assert excess(got[cu[b]:cu[b + 1]], ref, tol) <= 1.0, (b, n)


def test_fmha_profile_entry_point_matches_the_product_kernel(pkg, gpu):
    """mgpuBenchFusedMHAF16Profile (the benchmark's launch-loop library, not the kernel library) is the
    head_dim-64 kernel with clock stamps: the same output bits as mgpuFusedMHAF16, one record of ten
    counters per block, stamps in order."""
    import torch
    B, S, H, D = 2, 320, 3, 64
    g = torch.Generator(device=gpu).manual_seed(11)
    qkv = torch.randn((B, S, 3, H, D), device=gpu, generator=g).half()
    want = pkg.fused_mha(qkv)
    out = torch.zeros_like(want)
    blocks = B * H * ((S + 127) // 128)
    stamps = torch.zeros(blocks * 10, dtype=torch.int64, device=gpu)
    got = pkg.bench_loops().mgpuBenchFusedMHAF16Profile(qkv.data_ptr(), out.data_ptr(), B, S, H, D ** -0.5,
                                                        stamps.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert got == blocks
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    t = stamps.cpu().numpy().reshape(blocks, 10)
    entry, first, loop_end, stored, wall0, wall1 = (t[:, i] for i in range(6))
    assert np.all(entry < first) and np.all(first < loop_end) and np.all(loop_end < stored)
    assert np.all(wall1 > wall0)
    phases = t[:, 6:10].sum(axis=1)             # wait + scores + softmax + P.V of all tiles of the block
    assert np.all(phases > 0) and np.all(phases <= stored - entry)


@pytest.mark.parametrize("D,B,S,H,lens,causal,dtype", [
    (32, 2, 200, 3, None, False, "f16"),       # the reference's kernel list holds 32, 40, 80 next to 64 and 128
    (40, 2, 257, 2, [257, 90], False, "f16"),
    (40, 1, 384, 2, None, True, "f16"),         # causal in the 64-wide geometry
    (80, 2, 130, 3, [130, 1], False, "f16"),
    (80, 1, 300, 2, None, True, "bf16"),
    (96, 2, 96, 2, None, False, "bf16"),
    (8, 1, 70, 2, None, False, "f16"),          # the smallest head: one 16-byte chunk per row
    (120, 1, 129, 2, [100], True, "f16"),       # one chunk short of the 128-wide geometry
    (256, 2, 200, 2, None, False, "f16"),       # the widest head of the reference's kernel list: its own geometry
    (256, 1, 257, 2, [200], True, "f16"),
    (256, 2, 96, 3, [96, 33], False, "bf16"),
    (144, 2, 130, 2, [130, 7], False, "f16"),   # 144 and 160 of the list, inside the 256-wide geometry
    (160, 1, 300, 3, None, True, "f16"),
    (160, 2, 64, 2, None, False, "bf16"),
    (136, 1, 65, 1, None, False, "f16"),        # the first size past the 128-wide geometry
    (248, 1, 129, 2, [129], True, "f16"),       # one chunk short of the 256-wide geometry
    (80, 16, 512, 16, None, True, "f16"),       # 512 causal work items of two query blocks each, head size 80 inside 128
    (96, 32, 300, 8, None, True, "bf16"),       # 768 causal blocks handed out longest first, ragged last tile
])
def test_fmha_other_head_sizes(pkg, gpu, oracle, rng, D, B, S, H, lens, causal, dtype):
    """Head sizes between the tile geometries (64, 128, 256) run inside the next larger one: rows in
    memory stay D elements long (nothing is padded by the caller), the result is the
    attention over exactly D dimensions, and no byte outside [B, S, H*D] is written."""
    import torch
    qkv = rng.standard_normal((B, S, 3, H, D)).astype(np.float32)
    tq = torch.from_numpy(qkv).to(gpu).to(torch.float16 if dtype == "f16" else torch.bfloat16)
    bits = tq.view(torch.int16).cpu().numpy().view(np.uint16)
    out = torch.full((B * S + 1, H * D), 7.0, dtype=tq.dtype, device=gpu)  # one guard row behind the output
    tl = to_dev(np.asarray(lens, np.int32), gpu) if lens is not None else None
    pkg.fused_mha(tq, tl, causal=causal, out=out[:B * S].view(B, S, H * D))
    got = out.float().cpu().numpy()
    assert np.all(got[B * S] == 7.0)
    ref = oracle.fmha(bits.view(np.float16) if dtype == "f16" else bits, lens, causal=causal, bf16=dtype == "bf16")
    assert excess(got[:B * S].reshape(B, S, H * D), ref, TOL_F16 if dtype == "f16" else TOL_BF16) <= 1.0


def test_fmha_other_head_sizes_over_packed_rows(pkg, gpu, oracle, rng):
    import torch
    D, H, lens = 40, 2, [70, 0, 200]
    total = int(np.sum(lens))
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tq = torch.from_numpy(rng.standard_normal((total, 3, H, D)).astype(np.float32)).to(gpu).half()
    got = pkg.fused_mha_cu_seqlens(tq, to_dev(cu, gpu), 200).float().cpu().numpy()
    host = tq.cpu().numpy()
    for b, n in enumerate(lens):
        if n:
            assert excess(got[cu[b]:cu[b + 1]], oracle.fmha(host[cu[b]:cu[b + 1]][None])[0], TOL_F16) <= 1.0, b
