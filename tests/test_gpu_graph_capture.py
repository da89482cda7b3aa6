"""Entry points under HIP graph capture: a graph recorded from C-ABI calls must
replay to the same bits as the eager calls, on every replay, with new inputs
written and eager work run between the replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def replay_against_eager(torch, stream, call, refresh, result, replays=3):
    """call() enqueues on `stream`; refresh() rewrites the inputs; result() clones the output."""
    call()                      # plans, arenas and code objects exist before the capture starts
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            call()
    for _ in range(replays):
        refresh()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = result()
        call()
        stream.synchronize()
        assert torch.equal(got, result())


def test_streaming_kernels_and_attention_in_one_graph(pkg, gpu):
    import torch
    g = torch.Generator(device=gpu).manual_seed(5)
    st = torch.cuda.Stream()
    m, n = 300, 768
    a = torch.randn(m * n, device=gpu, generator=g)
    b = torch.randn(m * n, device=gpu, generator=g)
    gamma, beta = torch.randn(n, device=gpu, generator=g), torch.randn(n, device=gpu, generator=g)
    qkv = torch.randn((2, 200, 3, 4, 64), device=gpu, generator=g).half()
    lens = torch.tensor([200, 77], dtype=torch.int32, device=gpu)
    c, y = torch.empty_like(a), torch.empty((m, n), device=gpu)
    o = torch.empty((2, 200, 256), device=gpu, dtype=torch.float16)

    def call():
        pkg.add(a, b, out=c, stream=st)
        pkg.layer_norm(c.view(m, n), gamma, beta, out=y, stream=st)
        pkg.fused_mha(qkv, seqlens=lens, out=o, stream=st)

    def refresh():
        a.copy_(torch.randn(m * n, device=gpu, generator=g))
        qkv.copy_(torch.randn(qkv.shape, device=gpu, generator=g).half())

    replay_against_eager(torch, st, call, refresh, lambda: torch.cat([y.flatten(), o.flatten().float()]).clone())


def test_bert_layer_graph(pkg, gpu):
    import torch
    g = torch.Generator(device=gpu).manual_seed(6)
    st = torch.cuda.Stream()
    B, S, d, ffn, H = 2, 128, 256, 512, 4   # 256 tokens: the GEMMs may take either kernel
    h = lambda *s: (0.05 * torch.randn(*s, device=gpu, generator=g)).half()
    x = torch.randn((B, S, d), device=gpu, generator=g).half()
    P = [h(d, 3 * d), h(3 * d), h(d, d), h(d), (1 + h(d).float()).half(), h(d), h(d, ffn), h(ffn), h(ffn, d), h(d),
         (1 + h(d).float()).half(), h(d)]
    out = torch.empty_like(x)
    replay_against_eager(torch, st, lambda: pkg.bert_encoder_layer(x, *P, heads=H, out=out, stream=st),
                         lambda: x.copy_(torch.randn((B, S, d), device=gpu, generator=g).half()), lambda: out.clone())


def test_decoding_layer_graph(pkg, gpu):
    """The reference layer forks its weight casts to a side stream and joins them by events:
    both streams are captured."""
    import torch
    g = torch.Generator(device=gpu).manual_seed(7)
    st = torch.cuda.Stream()
    B, S, d, ffn, H = 2, 96, 256, 256, 2
    f = lambda *s: 0.05 * torch.randn(*s, device=gpu, generator=g)
    x = torch.randn((B, S, d), device=gpu, generator=g)
    W = [f(d, 3 * d), f(d, d), f(d), f(d, ffn), f(ffn), f(ffn, d), f(d)]
    out = torch.empty_like(x)
    lib = pkg.ops()

    def call():
        lib.mgpuLLMDecodingContextLayer(x.data_ptr(), *[w.data_ptr() for w in W], out.data_ptr(), B, S, d, ffn, H,
                                        True, True, True, st.cuda_stream)
        err = lib.mgpuOpsTakeLastError()
        assert err is None, err

    replay_against_eager(torch, st, call, lambda: x.copy_(torch.randn((B, S, d), device=gpu, generator=g)),
                         lambda: out.clone())


def test_bert_layer_captured_on_a_stream_without_arena(pkg, gpu):
    """First use of a stream inside a capture: the layer cannot keep an arena for the
    stream, so it allocates and frees inside the graph; replays still match eager."""
    import torch
    g = torch.Generator(device=gpu).manual_seed(8)
    B, S, d, ffn, H = 1, 64, 128, 256, 2
    h = lambda *s: (0.05 * torch.randn(*s, device=gpu, generator=g)).half()
    x = torch.randn((B, S, d), device=gpu, generator=g).half()
    P = [h(d, 3 * d), h(3 * d), h(d, d), h(d), (1 + h(d).float()).half(), h(d), h(d, ffn), h(ffn), h(ffn, d), h(d),
         (1 + h(d).float()).half(), h(d)]
    out = torch.empty_like(x)
    warm = torch.cuda.Stream()
    pkg.bert_encoder_layer(x, *P, heads=H, out=out, stream=warm)   # GEMM plans exist before the capture
    warm.synchronize()
    ref = out.clone()
    fresh = torch.cuda.Stream()                                     # no layer has run on this stream
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(fresh):
        with torch.cuda.graph(graph, stream=fresh):
            pkg.bert_encoder_layer(x, *P, heads=H, out=out, stream=fresh)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref)


def test_layer_arena_grows_and_is_reused(pkg, gpu, oracle):
    """A small layer, a larger one and the small one again on one stream: the arena of
    the stream grows once and the results do not depend on what ran before."""
    import torch
    g = torch.Generator(device=gpu).manual_seed(9)
    st = torch.cuda.Stream()

    def run(B, S, d, ffn, H, seed):
        gg = torch.Generator(device=gpu).manual_seed(seed)
        h = lambda *s: (0.05 * torch.randn(*s, device=gpu, generator=gg)).half()
        x = torch.randn((B, S, d), device=gpu, generator=gg).half()
        P = [h(d, 3 * d), h(3 * d), h(d, d), h(d), (1 + h(d).float()).half(), h(d), h(d, ffn), h(ffn), h(ffn, d),
             h(d), (1 + h(d).float()).half(), h(d)]
        out = pkg.bert_encoder_layer(x, *P, heads=H, stream=st)
        st.synchronize()
        return out

    small1 = run(1, 32, 128, 256, 2, 100)
    big = run(4, 128, 256, 1024, 4, 101)
    small2 = run(1, 32, 128, 256, 2, 100)
    assert torch.equal(small1, small2)
    assert torch.isfinite(big.float()).all()


def test_captured_layer_survives_a_growing_arena(pkg, gpu):
    """A layer captured on a stream that already keeps an arena, then a larger eager layer
    on the same stream (the kept arena is freed and replaced), then replays: the graph
    owns its own temporaries, so the replays still match the eager result."""
    import torch
    g = torch.Generator(device=gpu).manual_seed(10)
    st = torch.cuda.Stream()

    def params(d, ffn):
        h = lambda *s: (0.05 * torch.randn(*s, device=gpu, generator=g)).half()
        return [h(d, 3 * d), h(3 * d), h(d, d), h(d), (1 + h(d).float()).half(), h(d), h(d, ffn), h(ffn), h(ffn, d),
                h(d), (1 + h(d).float()).half(), h(d)]

    B, S, d, ffn, H = 1, 128, 128, 256, 2
    x = torch.randn((B, S, d), device=gpu, generator=g).half()
    P = params(d, ffn)
    out = torch.empty_like(x)
    pkg.bert_encoder_layer(x, *P, heads=H, out=out, stream=st)   # the stream now keeps a small arena
    st.synchronize()
    ref = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(st):
        with torch.cuda.graph(graph, stream=st):
            pkg.bert_encoder_layer(x, *P, heads=H, out=out, stream=st)
    xb = torch.randn((8, 128, 256), device=gpu, generator=g).half()
    big = pkg.bert_encoder_layer(xb, *params(256, 1024), heads=4, stream=st)  # grows the arena
    st.synchronize()
    assert torch.isfinite(big.float()).all()
    junk = torch.randn((64, 1024, 1024), device=gpu, generator=g)  # reuse whatever memory was returned
    for _ in range(3):
        out.zero_()
        junk.mul_(1.0001)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref)
