"""The hand-written MFMA GEMM (mgpuGemmMfmaF16 / BF16) against the oracle's GEMM,
through the C ABI: every epilogue, both types, every tile geometry, shapes from
one tile and one reduction step up to the BERT-base layer's, and the shapes it
must refuse."""
import numpy as np
import pytest

from conftest import to_dev

pytestmark = pytest.mark.gpu


def bf16_bits(t):
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def spacing_tol(ref, mant_bits, floor):
    """One spacing of the 16-bit result type at the reference's magnitude, plus a floor."""
    e = np.floor(np.log2(np.maximum(np.abs(ref), 2.0 ** -14)))
    return 2.0 ** (e - mant_bits) + floor


# M, K, N.  The launcher picks 128- or 96-column tiles and a reduction step of 32 or 64 from the shape (on the 256
# CUs of the test device): both widths and both steps are in the list, N = 672 and 96 only divide by 96, and
# (8192, 128, 672) is 448 tiles of 96 columns with the input rows fetched for two steps at a time.
SHAPES = [(128, 32, 128), (128, 64, 256), (256, 96, 384), (384, 160, 128), (256, 1024, 128), (256, 64, 96),
          (128, 32, 672), (512, 768, 768), (1024, 768, 3072), (4096, 768, 2304), (4096, 64, 3072), (8192, 128, 672)]


def epilogues(pkg, oracle, tb, b, tr, r):
    return [(dict(), dict()), (dict(bias=tb), dict(bias=b)), (dict(residual=tr), dict(residual=r)),
            (dict(bias=tb, act=pkg.ACT_RELU), dict(bias=b, act=oracle.ACT_RELU)),
            (dict(act=pkg.ACT_GELU), dict(act=oracle.ACT_GELU)),
            (dict(bias=tb, act=pkg.ACT_GELU), dict(bias=b, act=oracle.ACT_GELU)),
            (dict(bias=tb, residual=tr), dict(bias=b, residual=r))]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_gemm_mfma_f16(pkg, gpu, oracle, rng, M, K, N):
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16)
    r = rng.standard_normal((M, N)).astype(np.float16)
    tx, tw, tb, tr = [to_dev(t, gpu) for t in (x, w, b, r)]
    for kw, okw in epilogues(pkg, oracle, tb, b, tr, r):
        got = pkg.matmul_ex(tx, tw, kernel="mfma", **kw).cpu().numpy().astype(np.float32)
        ref = oracle.gemm(x, w, **okw)
        # fp32 accumulation, epilogue in fp32, one rounding: one fp16 spacing of the result
        err = np.abs(got - ref)
        assert np.all(err <= spacing_tol(ref, 10, 1e-3)), (sorted(kw), err.max())


@pytest.mark.parametrize("M,K,N", [(128, 32, 128), (256, 96, 384), (512, 768, 768), (4096, 64, 3072)])
def test_gemm_mfma_bf16(pkg, gpu, oracle, rng, M, K, N):
    import torch
    mk = lambda a: torch.from_numpy(a.astype(np.float32)).to(gpu).to(torch.bfloat16)
    tx, tw = mk(rng.standard_normal((M, K))), mk(rng.standard_normal((K, N)) / np.sqrt(K))
    tb, tr = mk(rng.standard_normal(N)), mk(rng.standard_normal((M, N)))
    x, w, b, r = [bf16_bits(t) for t in (tx, tw, tb, tr)]
    for kw, okw in epilogues(pkg, oracle, tb, b, tr, r):
        got = pkg.matmul_ex(tx, tw, kernel="mfma", **kw).float().cpu().numpy()
        ref = oracle.gemm(x, w, bf16=True, **okw)
        err = np.abs(got - ref)
        assert np.all(err <= spacing_tol(ref, 7, 4e-3)), (sorted(kw), err.max())


def test_gemm_mfma_matches_library_path(pkg, gpu, rng):
    """The measured choice behind mgpuMatmulExF16 may be either kernel: without an
    activation both round the same fp32 sums once, so they agree to the last bit
    wherever the two summation orders round alike, and to one spacing elsewhere
    (plus the fp32 noise of a 768-term sum where the terms cancel)."""
    M, K, N = 512, 768, 768
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16)
    tx, tw, tb = [to_dev(t, gpu) for t in (x, w, b)]
    a = pkg.matmul_ex(tx, tw, bias=tb).cpu().numpy().astype(np.float32)
    m = pkg.matmul_ex(tx, tw, bias=tb, kernel="mfma").cpu().numpy().astype(np.float32)
    assert np.all(np.abs(a - m) <= spacing_tol(m, 10, 1e-4))
    assert np.mean(a == m) > 0.99


def test_gemm_mfma_in_place_residual(pkg, gpu, oracle, rng):
    """The residual may be the output buffer itself (C == D), as the library path allows."""
    import torch
    M, K, N = 256, 64, 256
    x = rng.standard_normal((M, K)).astype(np.float16)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float16)
    r = rng.standard_normal((M, N)).astype(np.float16)
    tx, tw, out = to_dev(x, gpu), to_dev(w, gpu), to_dev(r, gpu)
    lib = pkg.ops()
    lib.mgpuGemmMfmaF16(tx.data_ptr(), tw.data_ptr(), None, out.data_ptr(), out.data_ptr(), M, N, K, 0, 0, 1,
                        torch.cuda.current_stream().cuda_stream)
    assert lib.mgpuOpsTakeLastError() is None
    torch.cuda.synchronize()
    ref = oracle.gemm(x, w, residual=r)
    assert np.all(np.abs(out.cpu().numpy().astype(np.float32) - ref) <= spacing_tol(ref, 10, 1e-3))


@pytest.mark.parametrize("M,K,N", [(100, 64, 128), (128, 48, 128), (128, 64, 72), (128, 0, 128)])
def test_gemm_mfma_refuses_other_shapes(pkg, gpu, M, K, N):
    import torch
    x = torch.zeros((M, max(K, 1)), dtype=torch.float16, device=gpu)[:, :K].contiguous()
    w = torch.zeros((max(K, 1), N), dtype=torch.float16, device=gpu)[:K].contiguous()
    with pytest.raises(pkg.MgpuError):
        pkg.matmul_ex(x, w, kernel="mfma")


def test_gemm_mfma_refuses_fp32_and_activation_with_residual(pkg, gpu):
    import torch
    x = torch.zeros((128, 32), dtype=torch.float16, device=gpu)
    w = torch.zeros((32, 128), dtype=torch.float16, device=gpu)
    r = torch.zeros((128, 128), dtype=torch.float16, device=gpu)
    with pytest.raises(pkg.MgpuError):
        pkg.matmul_ex(x, w, residual=r, act=pkg.ACT_RELU, kernel="mfma")
    with pytest.raises(KeyError):
        pkg.matmul_ex(x.float(), w.float(), kernel="mfma")


def test_gelu_erfc_form_tail(pkg, gpu, oracle):
    """x * Phi(x) on the negative tail, where 1 + erf cancels: a bias-only GEMM of
    zeros puts chosen values through the fused GELU."""
    import torch
    M, K, N = 128, 32, 128
    vals = np.linspace(-9.0, 9.0, N).astype(np.float16)
    x = torch.zeros((M, K), dtype=torch.float16, device=gpu)
    w = torch.zeros((K, N), dtype=torch.float16, device=gpu)
    got = pkg.matmul_ex(x, w, bias=to_dev(vals, gpu), act=pkg.ACT_GELU, kernel="mfma").cpu().numpy()
    ref = oracle.gemm(np.zeros((M, K), np.float16), np.zeros((K, N), np.float16), bias=vals, act=oracle.ACT_GELU)
    want = ref.astype(np.float16)
    # at most one unit in the last place of the fp16 result, subnormals included
    ulps = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    assert ulps.max() <= 1, ulps.max()


def test_forced_kernel_choice_in_a_fresh_process(gpu):
    """MGPU_GEMM_KERNEL=mfma / =library fix the path behind mgpuMatmulExF16; both give
    the same matrix up to one fp16 spacing."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, numpy as np, torch; sys.path.insert(0, %r)\n"
        "import __graft_entry__ as ge\n"
        "pkg = ge.load_package()\n"
        "g = torch.Generator(device='cuda:0').manual_seed(3)\n"
        "x = torch.randn((256, 256), device='cuda:0', generator=g).half()\n"
        "w = (torch.randn((256, 384), device='cuda:0', generator=g) / 16).half()\n"
        "b = torch.randn((384,), device='cuda:0', generator=g).half()\n"
        "y = pkg.matmul_ex(x, w, bias=b, act=pkg.ACT_GELU)\n"
        "np.save(sys.argv[1], y.cpu().numpy())\n" % root)
    outs = {}
    for mode in ("mfma", "library"):
        path = os.path.join("/tmp", "mgpu_forced_%s_%d.npy" % (mode, os.getpid()))
        env = dict(os.environ, MGPU_GEMM_KERNEL=mode)
        r = subprocess.run([sys.executable, "-c", code, path], env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        outs[mode] = np.load(path).astype(np.float32)
        os.remove(path)
    a, b = outs["mfma"], outs["library"]
    # the library path rounds before the GELU, the hand-written one after it: two spacings
    assert np.all(np.abs(a - b) <= 2 * spacing_tol(b, 10, 1e-3))


def test_gemm_mfma_refuses_a_misaligned_bias(pkg, gpu):
    import torch
    x = torch.zeros((128, 32), dtype=torch.float16, device=gpu)
    w = torch.zeros((32, 128), dtype=torch.float16, device=gpu)
    b = torch.zeros((130,), dtype=torch.float16, device=gpu)[1:129]   # 2 bytes off the 8-byte grid
    with pytest.raises(pkg.MgpuError):
        pkg.matmul_ex(x, w, bias=b, kernel="mfma")


def test_tuner_measures_outside_the_kernel_library(pkg, gpu):
    """The tuner that writes gemm_table.inc lives with the benchmark's launch loops
    (mgpuBenchTuneMatmulEx): it times the library on the ABI's [K, N] weight, the hand-written kernel and the
    library on a K-major weight on its own operands and reports all three; an unusable request reports -1; and
    the kernel library exports no tuning entry point."""
    import ctypes
    M, K, N = 256, 160, 384
    loops = pkg.bench_loops()
    times = (ctypes.c_float * 4)()
    index, version = ctypes.c_int32(-2), ctypes.c_int32(0)
    kept = loops.mgpuBenchTuneMatmulEx(1, M, N, K, 1, 0, 1, times, ctypes.byref(index), ctypes.byref(version))
    assert 0 <= kept <= 3
    library, mfma, k_major, best = list(times)
    assert library > 0 and mfma > 0 and k_major > 0
    assert 0 < best <= 1.1 * library                   # the best of the library's answers is no slower than its first
    assert index.value >= 0 and version.value > 0      # which library kernel that was
    assert (kept & 1) == (1 if mfma < 0.97 * library else 0)
    assert (kept >> 1) == (1 if k_major < 0.97 * min(library, mfma if kept & 1 else library) else 0)
    assert loops.mgpuBenchTuneMatmulEx(7, M, N, K, 1, 0, 1, None, None, None) == -1      # no such element type
    assert loops.mgpuBenchTuneMatmulEx(1, M, N, K, 1, 2, 1, None, None, None) == -1      # activation with a residual
    assert not hasattr(pkg.ops(), "mgpuMatmulExTune")


def test_library_gemm_captured_on_a_stream_that_has_no_workspace(pkg, gpu, oracle, rng):
    """The library's workspace belongs to a caller stream and is allocated on that
    stream's first GEMM outside a capture.  A GEMM captured on a stream that never ran
    one must not allocate: it takes an algorithm that needs no workspace, and every
    replay gives the eager result's matrix (fp32: always the library's kernel)."""
    import torch
    M, K, N = 96, 200, 72
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    tx, tw, tb = [to_dev(t, gpu) for t in (x, w, b)]
    out = torch.zeros((M, N), device=gpu)
    lib = pkg.ops()
    st = torch.cuda.Stream()                    # fresh: no workspace behind it

    def call():
        lib.mgpuMatmulExF32(tx.data_ptr(), tw.data_ptr(), tb.data_ptr(), out.data_ptr(), None, M, N, K, 1, 0, 0,
                            st.cuda_stream)
        assert lib.mgpuOpsTakeLastError() is None

    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(graph, stream=st):
            call()
    ref = oracle.gemm(x, w, b)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.abs(out.cpu().numpy() - ref).max() <= 1.2e-5
    call()                                      # eager, after the capture: may now allocate the workspace
    st.synchronize()
    assert np.abs(out.cpu().numpy() - ref).max() <= 1.2e-5
