"""Seeded random shapes through every operator, against double-precision torch on the CPU.

The other GPU tests pin chosen shapes to the oracle bit for bit or to one unit in the last place; this one walks
shapes nobody chose (sizes around powers of two, tiny ones, ragged ones, every dtype and option of the front end)
and looks for gross errors: a wrong index, an element left unwritten, a store outside the output. Every output
is a window of a larger buffer: the window starts as NaN, so an element the kernel skips shows, and the 256 elements
on either side hold a sentinel that must survive. Tolerances are the largest error relative to the largest expected
value: 3e-3 for fp16 results, 2e-2 for bf16, 2e-5 for fp32 (twice that after a norm or an element-wise function,
more where stated at the case).
"""
import math
import random

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

PAD = 256


def guarded(shape, dtype):
    n = 1
    for s in shape:
        n *= s
    buf = torch.full((PAD + n + PAD,), 777.0 if dtype.is_floating_point else 77, dtype=dtype, device="cuda")
    out = buf[PAD:PAD + n].view(shape)
    if dtype.is_floating_point:
        out.fill_(float("nan"))
    return buf, out


def check_guard(buf, n, what):
    lo, hi = buf[:PAD].cpu(), buf[PAD + n:].cpu()
    v = 777.0 if buf.dtype.is_floating_point else 77
    if not (bool((lo == v).all()) and bool((hi == v).all())):
        raise AssertionError("stored outside the output: " + what)


def compare(got, want, tol, what):
    got, want = got.cpu().double(), want.double()
    if got.shape != want.shape:
        raise AssertionError("shape %s, expected %s: %s" % (tuple(got.shape), tuple(want.shape), what))
    if got.numel() == 0:
        return
    if torch.isnan(got).any():
        raise AssertionError("%d elements NaN or not written: %s" % (int(torch.isnan(got).sum()), what))
    scale = want.abs().max().clamp_min(1e-30)
    err = ((got - want).abs().max() / scale).item()
    if err > tol:
        idx = (got - want).abs().argmax().item()
        raise AssertionError("%s: error %.3g above %.3g at element %d: got %g, expected %g"
                             % (what, err, tol, idx, got.flatten()[idx], want.flatten()[idx]))


# set by the test for each operator: the random streams, the size class, the package under test
rnd = random.Random(0)
g = torch.Generator()
BIG = False
ops = hexmi_pkg = None


def pick(*choices):
    return rnd.choice(choices)


def dim(lo, hi, specials=()):
    r = rnd.random()
    if specials and r < 0.35:
        return rnd.choice(specials)
    if r < 0.6:
        return rnd.randint(lo, min(hi, lo + 40))
    return rnd.randint(lo, hi)


TOL = {torch.float16: 3e-3, torch.bfloat16: 2e-2, torch.float32: 2e-5}


def case_softmax():
    dt = pick(torch.float32, torch.float16, torch.bfloat16)
    rows = dim(1, 3000 if BIG else 300, (1, 2, 63, 64, 65, 128, 255, 256, 257))
    cols = dim(1, 40000 if BIG else 5000, (1, 2, 3, 7, 8, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193, 16384, 20000, 33000))
    bc = pick(0, 0, 0, 64, 128, 1000)
    what = "softmax %s rows=%d cols=%d block_cols=%d" % (dt, rows, cols, bc)
    print(what, flush=True)
    x = (torch.randn(rows, cols, generator=g) * 3).to(dt)
    buf, out = guarded((rows, cols), dt)
    ops.softmax(x.cuda(), out=out, block_cols=bc)
    torch.cuda.synchronize()
    check_guard(buf, rows * cols, what)
    compare(out, F.softmax(x.double(), dim=-1), TOL[dt], what)


def case_norms():
    dt = pick(torch.float16, torch.bfloat16, torch.float32)
    rows = dim(1, 300, (1, 2, 63, 64, 65, 127, 128, 129, 256))
    cols = dim(1, 5000, (1, 2, 3, 7, 8, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193, 16384, 20000))
    layer = rnd.random() < 0.5
    bc = pick(0, 0, 0, 64, 1000)
    what = "%s %s rows=%d cols=%d block_cols=%d" % ("layer_norm" if layer else "rms_norm", dt, rows, cols, bc)
    print(what, flush=True)
    x = (torch.randn(rows, cols, generator=g) * 2 + 0.5).to(dt)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dt)
    b = (0.1 * torch.randn(cols, generator=g)).to(dt)
    buf, out = guarded((rows, cols), dt)
    if layer:
        mb, mean = guarded((rows,), torch.float32)
        rb, rstd = guarded((rows,), torch.float32)
        ops.layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-5, out=out, mean=mean, rstd=rstd, block_cols=bc)
        torch.cuda.synchronize()
        check_guard(mb, rows, what); check_guard(rb, rows, what)
        want = F.layer_norm(x.double(), (cols,), w.double(), b.double(), 1e-5)
        compare(mean, x.double().mean(-1), 1e-4, what + " mean")
        compare(rstd, 1 / torch.sqrt(x.double().var(-1, unbiased=False) + 1e-5), 1e-4, what + " rstd")
    else:
        ops.rms_norm(x.cuda(), w.cuda(), 1e-5, out=out, block_cols=bc)
        torch.cuda.synchronize()
        xd = x.double()
        want = xd * torch.rsqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * w.double()
    check_guard(buf, rows * cols, what)
    compare(out, want, TOL[dt] * 2, what)


def case_gemm():
    dt = pick(torch.float16, torch.float16, torch.bfloat16, torch.float32)
    M = dim(1, 2500 if BIG else 700, (1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513))
    N = dim(1, 2500 if BIG else 700, (1, 2, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 512, 520))
    K = dim(1, 5000 if BIG else 2100, (1, 2, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 256, 264, 512, 1024, 2048))
    tb = rnd.random() < 0.4
    odt = torch.float32 if dt == torch.float32 or rnd.random() < 0.25 else dt
    use_bias, use_res = rnd.random() < 0.3, rnd.random() < 0.3
    what = "gemm %s M=%d N=%d K=%d trans_b=%s out=%s bias=%s res=%s" % (dt, M, N, K, tb, odt, use_bias, use_res)
    print(what, flush=True)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(dt)
    b = (torch.rand((N, K) if tb else (K, N), generator=g) * 2 - 1).to(dt)
    bias = torch.randn(N, generator=g).to(odt) if use_bias else None
    res = torch.randn(M, N, generator=g).to(odt) if use_res else None
    buf, out = guarded((M, N), odt)
    ops.matmul(a.cuda(), b.cuda(), out=out, trans_b=tb, bias=None if bias is None else bias.cuda(), residual=None if res is None else res.cuda())
    torch.cuda.synchronize()
    check_guard(buf, M * N, what)
    want = a.double() @ (b.double().T if tb else b.double())
    if bias is not None: want = want + bias.double()
    if res is not None: want = want + res.double()
    # 16-bit operands with an fp32 result: the products are exact, the fp32 sums of up to 5000 terms are not
    compare(out, want, 1e-4 if dt != torch.float32 and odt == torch.float32 else 3e-5 if dt == torch.float32 else TOL[odt], what)


def case_w8():
    M = dim(1, 300, (1, 2, 3, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 80, 96, 97, 127, 128, 129, 255, 256, 257))
    N = dim(1, 30000 if BIG else 3000, (1, 15, 16, 17, 47, 48, 49, 255, 256, 257, 1000, 4096, 11008, 12288, 12289, 16384, 24577))
    K = dim(1, 12000 if BIG else 3000, (16, 32, 48, 64, 80, 128, 192, 256, 320, 512, 768, 832, 1024, 1088, 2048, 2112, 4096, 4160, 5120, 8192, 8256, 11008))
    if rnd.random() < 0.7:
        K = max(16, K // 16 * 16) if rnd.random() < 0.5 else max(64, K // 64 * 64)
    if N * K > 60e6:
        N = max(1, int(60e6 // K))
    if M * N * K > 3e10:
        M = max(1, int(3e10 // (N * K)))
    mode = pick("plain", "plain", "plain", "zp", "zp", "pt", "pt_zp", "packed", "ws")
    if mode == "packed":
        K = pick(1024, 2048, 3072, 4096)
    what = "w8a16 %s M=%d N=%d K=%d" % (mode, M, N, K)
    print(what, flush=True)
    a = torch.randn(M, K, generator=g).half()
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    ns = 1 if mode in ("pt", "pt_zp") else N
    s = (0.001 + 0.019 * torch.rand(ns, generator=g)).half()
    zp = torch.randint(-128, 128, (ns,), generator=g, dtype=torch.int8) if mode in ("zp", "pt_zp") else None
    buf, out = guarded((M, N), torch.float16)
    if mode == "packed":
        wp = ops.pack_w8(w.cuda())
        ops.w8a16_matmul_packed(a.cuda(), wp, s.cuda(), out=out)
    elif mode == "ws":
        lib = hexmi_pkg.lib()
        ad, wd, sd = a.cuda(), w.cuda(), s.cuda()
        rc = lib.hexmi_gemm_w8a16(M, N, K, ad.data_ptr(), wd.data_ptr(), sd.data_ptr(), out.data_ptr(), None)
        if rc != 0:
            raise AssertionError("status %d: %s" % (rc, what))
    else:
        ops.w8a16_matmul(a.cuda(), w.cuda(), s.cuda(), out=out, zero_points=None if zp is None else zp.cuda())
    torch.cuda.synchronize()
    check_guard(buf, M * N, what)
    wf = w.float()
    if zp is not None:
        wf = wf - zp.float()[:, None] if ns == N else wf - float(zp[0])
    wf = wf * (s.float()[:, None] if ns == N else float(s[0]))
    want = a.float() @ wf.T
    compare(out, want, 3e-3, what)


def case_flash():
    dt = pick(torch.float16, torch.float16, torch.bfloat16, torch.float32)
    # the kernels' own head sizes, narrower and wider ones on padded tiles, and one for the row-wise kernel
    D = pick(64, 128, 128, 8, 40, 80, 96, 160, 192, 256, 20) if dt != torch.float32 else pick(64, 128, 4, 36, 80, 100, 10)
    Z, H = pick(1, 2, 3), pick(1, 2, 3, 5, 8, 9)
    if D > 128 or D in (10, 20):
        H = min(H, 3)
    S = dim(1, 2600 if BIG else 900, (1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 383, 384, 512, 640, 1024, 1100))
    causal = rnd.random() < 0.6
    what = "flash %s Z=%d H=%d S=%d D=%d causal=%s" % (dt, Z, H, S, D, causal)
    print(what, flush=True)
    q, k, v = (torch.randn(Z, H, S, D, generator=g).to(dt) for _ in range(3))
    buf, out = guarded((Z, H, S, D), dt)
    ops.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal, out=out)
    torch.cuda.synchronize()
    check_guard(buf, Z * H * S * D, what)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal)
    compare(out, want, {torch.float16: 4e-3, torch.bfloat16: 2.5e-2, torch.float32: 1e-4}[dt], what)


def case_attention():
    dt = pick(torch.float16, torch.bfloat16, torch.float32)
    D = pick(64, 128, 32, 80, 112) if dt != torch.float32 else pick(64, 128, 36, 80)
    B = pick(1, 2, 5, 9)
    Sq = dim(1, 2000 if BIG else 600, (1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257))
    Skv = dim(1, 2000 if BIG else 600, (1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257))
    masked = rnd.random() < 0.6
    what = "attention %s B=%d Sq=%d Skv=%d D=%d mask=%s" % (dt, B, Sq, Skv, D, masked)
    print(what, flush=True)
    q = torch.randn(B, Sq, D, generator=g).to(dt)
    k = torch.randn(B, Skv, D, generator=g).to(dt)
    v = torch.randn(B, Skv, D, generator=g).to(dt)
    mask = None
    if masked:
        mask = torch.randn(B, Sq, Skv, generator=g)
        drop = torch.rand(B, Sq, Skv, generator=g) < 0.2
        drop[:, :, rnd.randrange(Skv)] = False
        mask = torch.where(drop, torch.tensor(float("-inf")), mask).to(dt)
    buf, out = guarded((B, Sq, D), dt)
    ops.attention(q.cuda(), k.cuda(), v.cuda(), mask=None if mask is None else mask.cuda(), out=out)
    torch.cuda.synchronize()
    check_guard(buf, B * Sq * D, what)
    sc = q.double() @ k.double().transpose(1, 2) / math.sqrt(D)
    if mask is not None:
        sc = sc + mask.double()
    want = torch.softmax(sc, dim=-1) @ v.double()
    compare(out, want, {torch.float16: 4e-3, torch.bfloat16: 2.5e-2, torch.float32: 1e-4}[dt], what)


def case_elementwise():
    dt = pick(torch.float16, torch.bfloat16, torch.float32)
    n = dim(1, 200000, (1, 2, 7, 8, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 65535, 65536, 65537, 1 << 20))
    kind = pick("unary", "binary", "block_sum", "rope")
    if kind == "unary":
        op = pick(*ops.UNARY_OPS)
        what = "unary %s %s n=%d" % (op, dt, n)
        print(what, flush=True)
        x = torch.randn(n, generator=g)
        if op == "rsqrt":
            x = x.abs() + 0.1
        x = x.to(dt)
        buf, out = guarded((n,), dt)
        ops.unary(op, x.cuda(), out=out)
        torch.cuda.synchronize()
        xd = x.double()
        want = {"gelu_tanh": lambda: F.gelu(xd, approximate="tanh"), "silu": lambda: F.silu(xd), "rsqrt": lambda: torch.rsqrt(xd),
                "sin": lambda: torch.sin(xd), "cos": lambda: torch.cos(xd), "exp": lambda: torch.exp(xd)}[op]()
        check_guard(buf, n, what)
        compare(out, want, TOL[dt] * 2, what)
    elif kind == "binary":
        op = pick(*ops.BINARY_OPS)
        what = "binary %s %s n=%d" % (op, dt, n)
        print(what, flush=True)
        a = torch.randn(n, generator=g).to(dt)
        b = (torch.randn(n, generator=g).abs() + 0.5).to(dt)
        buf, out = guarded((n,), dt)
        ops.binary(op, a.cuda(), b.cuda(), out=out)
        torch.cuda.synchronize()
        ad, bd = a.double(), b.double()
        want = {"add": ad + bd, "sub": ad - bd, "mul": ad * bd, "div": ad / bd}[op]
        check_guard(buf, n, what)
        compare(out, want, TOL[dt] * 2, what)
    elif kind == "block_sum":
        block = pick(None, 1, 7, 64, 1000, 4096, 100000)
        what = "block_sum %s n=%d block=%s" % (dt, n, block)
        print(what, flush=True)
        x = torch.randn(n, generator=g).to(dt)
        bl = n if block is None else block
        programs = (n + bl - 1) // bl
        buf, out = guarded((programs,), dt)
        ops.block_sum(x.cuda(), block, out=out)
        torch.cuda.synchronize()
        xd = torch.cat([x.double(), torch.zeros(programs * bl - n, dtype=torch.double)]).view(programs, bl).sum(-1)
        check_guard(buf, programs, what)
        got, w = out.cpu().double(), xd
        err = (got - w).abs().max().item()
        lim = {torch.float16: 2e-3, torch.bfloat16: 1.6e-2, torch.float32: 1e-5}[dt] * max(1.0, w.abs().max().item()) + {torch.float16: 1e-3, torch.bfloat16: 8e-3, torch.float32: 1e-6}[dt] * math.sqrt(bl)
        if torch.isnan(got).any() or err > lim:
            raise AssertionError("%s: error %.3g above %.3g" % (what, err, lim))
    else:
        Bt, S, H, Fe = pick(1, 2, 3), dim(1, 300, (1, 63, 64, 65)), pick(1, 2, 5, 8, 32), pick(2, 4, 6, 8, 16, 32, 64, 128, 130, 256)
        what = "rope %s B=%d S=%d H=%d F=%d" % (dt, Bt, S, H, Fe)
        print(what, flush=True)
        x = torch.randn(Bt, S, H, Fe, generator=g).to(dt)
        buf, out = guarded((Bt, S, H, Fe), dt)
        ops.rope(x.cuda(), 10000.0, out=out)
        torch.cuda.synchronize()
        pos = torch.arange(S, dtype=torch.double)
        inv = 1.0 / (10000.0 ** (torch.arange(0, Fe, 2, dtype=torch.double) / Fe))
        ang = pos[:, None] * inv[None, :]
        c, s_ = torch.cos(ang)[None, :, None, :], torch.sin(ang)[None, :, None, :]
        xd = x.double()
        x0, x1 = xd[..., 0::2], xd[..., 1::2]
        want = torch.stack([x0 * c - x1 * s_, x0 * s_ + x1 * c], dim=-1).flatten(-2)
        check_guard(buf, x.numel(), what)
        compare(out, want, TOL[dt] * 2, what)


def case_ams():
    dt = pick(torch.float16, torch.bfloat16, torch.float32)
    M, K, N = dim(1, 300, (1, 31, 32, 33, 64)), dim(1, 300, (1, 31, 32, 33, 64)), dim(1, 1024, (1, 31, 32, 33, 512, 1023, 1024))
    fused = pick(None, True, False)
    what = "add_matmul_softmax %s M=%d K=%d N=%d fused=%s" % (dt, M, K, N, fused)
    print(what, flush=True)
    x = torch.randn(M, K, generator=g).to(dt) * 0.3
    y = torch.randn(M, K, generator=g).to(dt) * 0.3
    z = torch.randn(K, N, generator=g).to(dt) * 0.3
    buf, out = guarded((M, N), dt)
    ops.add_matmul_softmax(x.cuda(), y.cuda(), z.cuda(), out=out, fused=fused)
    torch.cuda.synchronize()
    check_guard(buf, M * N, what)
    # the sum x + y is rounded to the operand type before the product, as in the reference graph
    want = F.softmax((x + y).double() @ z.double(), dim=-1)
    compare(out, want, {torch.float16: 1.5e-2, torch.bfloat16: 8e-2, torch.float32: 1e-4}[dt], what)


CASES = {"softmax": case_softmax, "norms": case_norms, "gemm": case_gemm, "w8a16": case_w8, "flash_attention": case_flash,
         "attention": case_attention, "elementwise": case_elementwise, "add_matmul_softmax": case_ams}


@pytest.mark.parametrize("big", [False, True], ids=["small", "large"])
@pytest.mark.parametrize("name", list(CASES))
def test_random_shapes(hexmi, name, big):
    global rnd, g, BIG, ops, hexmi_pkg
    hexmi_pkg, ops = hexmi, hexmi.ops
    seed = sorted(CASES).index(name) * 2 + int(big) + 100
    rnd, BIG = random.Random(seed), big
    g = torch.Generator().manual_seed(seed)
    for _ in range(120 if big else 300):
        CASES[name]()
