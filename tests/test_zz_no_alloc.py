"""mgpuBertEncoderLayerF16NoAlloc (temporaries in the library's fixed device
array, nothing allocated) against mgpuBertEncoderLayerF16 and the oracle, on
two calls in a row, the second on a smaller input, through the C ABI.

The two entry points may run different GEMM kernels (the existing one may take
the library's), which round fp16 intermediates differently, so equality is to
the layer's parity bound, written below; both are also held to the oracle."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu


def layer_tol(ref):
    # fp16 output of an O(1..4) tensor after ~6 fp16-rounded stages; floor = one fp16
    # spacing of the residual stream
    return 5e-3 + 4e-3 * np.abs(ref)


def _params(rng, d, ffn):
    h16 = lambda *s: (0.02 * rng.standard_normal(s)).astype(np.float16)
    gam = lambda: (1 + 0.02 * rng.standard_normal(d)).astype(np.float16)
    return [h16(d, 3 * d), h16(3 * d), h16(d, d), h16(d), gam(), h16(d), h16(d, ffn), h16(ffn), h16(ffn, d),
            h16(d), gam(), h16(d)]


def test_no_alloc_layer_matches_allocating_entry_point(pkg, gpu, oracle):
    import torch
    rng = np.random.Generator(np.random.PCG64(20247))
    d, ffn, H = 768, 3072, 12
    P = _params(rng, d, ffn)
    Pd = [to_dev(p, gpu) for p in P]
    # the first call fills most of the array (36 of 48 MiB); the second, smaller one
    # finds the first call's contents in it and must not be disturbed by them.  The
    # pair runs twice: by the second round every kernel has been launched once (the
    # runtime loads code on first use), so the device's free memory must not move.
    for round_ in range(2):
        for (B, S, masked) in ((32, 128, False), (3, 128, True)):
            x = rng.standard_normal((B, S, d)).astype(np.float16)
            lens = rng.integers(1, S + 1, B).astype(np.int32) if masked else None
            xd = to_dev(x, gpu)
            ld = to_dev(lens, gpu) if masked else None
            out = torch.empty_like(xd)
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            got = pkg.bert_encoder_layer(xd, *Pd, heads=H, seqlens=ld, out=out, no_alloc=True)
            torch.cuda.synchronize()
            if round_ == 1:
                assert torch.cuda.mem_get_info()[0] == free_before, "the no-alloc entry point changed the device's free memory"
            got = got.cpu().numpy().astype(np.float32)
            want = pkg.bert_encoder_layer(xd, *Pd, heads=H, seqlens=ld).cpu().numpy().astype(np.float32)
            ref = oracle.bert_layer_f16(x, *P, heads=H, seqlens=lens)
            assert np.all(np.isfinite(got))
            assert np.all(np.abs(got - want) <= layer_tol(want)), np.abs(got - want).max()
            assert np.abs(got - want).mean() <= 5e-4
            assert np.all(np.abs(got - ref) <= layer_tol(ref)), np.abs(got - ref).max()
            assert np.abs(got - ref).mean() <= 5e-4


def test_no_alloc_layer_rejects_what_does_not_fit(pkg, gpu):
    import torch
    rng = np.random.Generator(np.random.PCG64(3))
    d, ffn, H = 768, 3072, 12
    Pd = [to_dev(p, gpu) for p in _params(rng, d, ffn)]
    x = torch.zeros((44, 128, d), dtype=torch.float16, device=gpu)  # 49.5 MiB of temporaries
    with pytest.raises(pkg.MgpuError, match="fixed scratch holds"):
        pkg.bert_encoder_layer(x, *Pd, heads=H, no_alloc=True)
    x = torch.zeros((1, 100, d), dtype=torch.float16, device=gpu)   # 100 tokens: not a multiple of 128
    with pytest.raises(pkg.MgpuError, match="multiple of 128"):
        pkg.bert_encoder_layer(x, *Pd, heads=H, no_alloc=True)
