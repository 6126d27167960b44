"""Every operator family captured into a HIP graph and replayed several times on changing inputs must give what the
eager launch gives: the benchmark times graph replays, and serving loops replay graphs. Between replays the test does
eager work and synchronises, and every replay is checked (a node that only works on the first replay would pass a
single comparison)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _cases(hexmi):
    g = torch.Generator().manual_seed(77)

    def r(*shape, dtype=torch.float16, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()

    w8 = torch.randint(-127, 128, (512, 1024), generator=g, dtype=torch.int8).cuda()
    w8k = torch.randint(-127, 128, (320, 8192), generator=g, dtype=torch.int8).cuda()      # a long K: summed over K parts
    sck = (0.001 + 0.01 * torch.rand(320, generator=g)).half().cuda()
    sc = (0.001 + 0.01 * torch.rand(512, generator=g)).half().cuda()
    wn, bn = r(4096), r(4096)
    bmat, bias, zs = r(768, 512, scale=0.05), r(512), r(64, 96, dtype=torch.float32)
    k4, v4 = r(2, 4, 512, 128), r(2, 4, 512, 128)
    k3, v3, mask = r(4, 384, 128), r(4, 384, 128), r(4, 256, 384)
    # name, the input that changes between replays, the launch (x, out) -> None, the output buffer
    return [
        ("softmax", r(512, 1024, dtype=torch.float32), lambda x, o: hexmi.softmax(x, out=o), None),
        ("rms_norm", r(256, 4096), lambda x, o: hexmi.rms_norm(x, wn, 1e-5, out=o), None),
        ("layer_norm", r(256, 4096), lambda x, o: hexmi.layer_norm(x, wn, bn, 1e-5, out=o), None),
        ("linear", r(384, 768), lambda x, o: hexmi.matmul(x, bmat, out=o, bias=bias, residual=o), (384, 512)),
        ("gemm_f32out", r(384, 768), lambda x, o: hexmi.matmul(x, bmat, out=o), ((384, 512), torch.float32)),
        ("w8a16_m1", r(1, 1024), lambda x, o: hexmi.w8a16_matmul(x, w8, sc, out=o), (1, 512)),
        ("w8a16_m16", r(16, 1024), lambda x, o: hexmi.w8a16_matmul(x, w8, sc, out=o), (16, 512)),
        ("w8a16_m64", r(64, 1024), lambda x, o: hexmi.w8a16_matmul(x, w8, sc, out=o), (64, 512)),
        ("w8a16_m200", r(200, 1024), lambda x, o: hexmi.w8a16_matmul(x, w8, sc, out=o), (200, 512)),
        ("w8a16_k_parts", r(96, 8192), lambda x, o: hexmi.w8a16_matmul(x, w8k, sck, out=o), (96, 320)),
        ("softmax_split_rows", r(4, 65536, dtype=torch.float32), lambda x, o: hexmi.softmax(x, out=o), None),
        ("layer_norm_column_blocks", r(64, 4096), lambda x, o: hexmi.layer_norm(x, wn, bn, 1e-5, out=o, block_cols=1024), None),
        ("flash_causal", r(2, 4, 512, 128), lambda x, o: hexmi.flash_attention(x, k4, v4, 128 ** -0.5, True, out=o), None),
        ("attention_masked", r(4, 256, 128), lambda x, o: hexmi.attention(x, k3, v3, mask, out=o), None),
        ("gelu", r(1000, 333), lambda x, o: hexmi.gelu(x, out=o), None),
        ("rope", r(2, 64, 4, 64, dtype=torch.float32), lambda x, o: hexmi.rope(x, 10000.0, out=o), None),
        ("block_sum_two_pass", r(1 << 20, dtype=torch.float32), lambda x, o: hexmi.block_sum(x, out=o), (1,)),
        ("add_matmul_softmax_fused", r(48, 64, dtype=torch.float32),
         lambda x, o: hexmi.add_matmul_softmax(x, x, zs, out=o, fused=True), (48, 96)),
        ("add_matmul_softmax_three", r(48, 64, dtype=torch.float32),
         lambda x, o: hexmi.add_matmul_softmax(x, x, zs, out=o, fused=False), (48, 96)),
    ]


def test_graph_replays_match_eager(hexmi):
    g = torch.Generator().manual_seed(78)
    for name, x, launch, out_spec in _cases(hexmi):
        if out_spec is None:
            shape, dtype = tuple(x.shape), x.dtype
        elif isinstance(out_spec[0], tuple):
            shape, dtype = out_spec
        else:
            shape, dtype = out_spec, x.dtype
        is_inplace_residual = name == "linear"
        out = torch.zeros(shape, dtype=dtype, device="cuda")
        eager = torch.zeros_like(out)
        launch(x, eager)                                              # warm-up outside the capture
        torch.cuda.synchronize()
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                launch(x, out)
        for replay in range(3):
            fresh = (torch.randn(x.shape, generator=g) * (0.5 + replay)).to(x.dtype)
            x.copy_(fresh.cuda())                                     # eager work between the replays
            start = (torch.randn(shape, generator=g) * 0.1).to(dtype).cuda() if is_inplace_residual else None
            if start is not None:
                out.copy_(start)
                eager.copy_(start)
            launch(x, eager)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), "%s: replay %d differs from the eager launch" % (name, replay)
            assert torch.isfinite(out.float()).all(), name


def test_calls_on_two_streams_do_not_interfere(hexmi):
    # the library keeps no state between calls (the one documented exception is hexmi_block_sum_static): launches that
    # overlap on two streams give what they give alone
    g = torch.Generator().manual_seed(79)
    a = torch.randn(1024, 1024, generator=g).half().cuda()
    b = torch.randn(1024, 1024, generator=g).half().cuda()
    x = torch.randn(4096, 1024, generator=g).cuda()
    q, k, v = (torch.randn(1, 8, 1024, 128, generator=g).half().cuda() for _ in range(3))
    xs = torch.randn(1 << 20, generator=g).cuda()
    want = (hexmi.matmul(a, b), hexmi.softmax(x), hexmi.flash_attention(q, k, v, 128 ** -0.5, True), hexmi.block_sum(xs))
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for _ in range(5):
        with torch.cuda.stream(s1):
            c = hexmi.matmul(a, b)
            o = hexmi.flash_attention(q, k, v, 128 ** -0.5, True)
        with torch.cuda.stream(s2):
            y = hexmi.softmax(x)
            t = hexmi.block_sum(xs)
        torch.cuda.synchronize()
        for got, ref in zip((c, y, o, t), want):
            assert torch.equal(got, ref)


def test_operators_through_the_dispatcher(hexmi):
    # the route tracing needs: the public operators as torch.ops.hexmi.* calls, same results bit for bit
    g = torch.Generator().manual_seed(80)
    x = torch.randn(64, 1024, generator=g).half().cuda()
    w = (1 + 0.1 * torch.randn(1024, generator=g)).half().cuda()
    b = torch.randn(1024, 256, generator=g).half().cuda()
    direct = (hexmi.softmax(x), hexmi.rms_norm(x, w, 1e-5), hexmi.layer_norm(x, w, w, 1e-5), hexmi.matmul(x, b))
    previous = hexmi.through_dispatcher(True)
    try:
        routed = (hexmi.softmax(x), hexmi.rms_norm(x, w, 1e-5), hexmi.layer_norm(x, w, w, 1e-5), hexmi.matmul(x, b))
    finally:
        hexmi.through_dispatcher(previous)
    for d, r in zip(direct, routed):
        assert torch.equal(d, r)
