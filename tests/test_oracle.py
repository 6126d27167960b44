"""Pins the CPU oracle (oracle/hexmi_oracle.c) against the library calls the reference's own tests use as
their oracle (torch CPU ops), at the reference's shapes, plus closed forms and invariants chosen so that a
dropped term, a wrong index or a transposed operand fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import torch_cpu


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


def _bf16_bits(t):
    return t.view(torch.int16).numpy().view(np.uint16)


def _ulp16(a, b):
    """Largest distance, in units of the 16-bit format's last place, between two fp16/bf16 tensors."""
    def key(t):
        i = t.view(torch.int16).int()
        return torch.where(i < 0, -(i & 0x7FFF), i)      # sign-magnitude -> monotone integer
    return (key(a) - key(b)).abs().max().item()


def _close16(a, b, atol):
    """Every element within one unit in the last place, or within atol where the value is a cancellation
    residue (x_hat*w + b near zero) whose fp32 library result carries the rounding of its larger terms."""
    def key(t):
        i = t.view(torch.int16).int()
        return torch.where(i < 0, -(i & 0x7FFF), i)
    ok = ((key(a) - key(b)).abs() <= 1) | ((a.float() - b.float()).abs() <= atol)
    return bool(ok.all())


def _bits_bf16(a):
    return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)


# ---------------------------------------------------------------- conversions
def test_f16_conversion_matches_numpy(oracle):
    rng = np.random.default_rng(0)
    vals = (rng.standard_normal(5000) * np.exp(rng.uniform(-20, 12, 5000))).astype(np.float32)
    vals = np.concatenate([vals, np.float32([0, -0.0, 65504, 65519.996, 65520, 2 ** -25, 2 ** -24, 5.96e-8, 1e-8])])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16_bits(float(v)) for v in vals], np.uint16)
    assert (want == got).all()


def test_bf16_conversion_matches_torch(oracle):
    g = torch.Generator().manual_seed(1)
    vals = torch.randn(4000, generator=g) * torch.exp(torch.rand(4000, generator=g) * 40 - 20)
    want = _bf16_bits(vals.to(torch.bfloat16))
    got = np.array([oracle.f32_to_bf16_bits(float(v)) for v in vals], np.uint16)
    assert (want == got).all()


# -------------------------------------------------------------------- softmax
@pytest.mark.parametrize("dtype,atol", [(torch.float32, 1e-7), (torch.float16, 0.0)])
@pytest.mark.parametrize("shape", [(128, 128), (4, 65536), (37, 513)])
def test_softmax_vs_torch(oracle, dtype, atol, shape):
    # reference shapes: 128x128 (test_softmax.py:21-23), 4x65536 (test_softmax_scf_multithread.py:19-24)
    g = torch.Generator().manual_seed(0)
    x = torch.rand(*shape, generator=g).to(dtype)
    got = _t(oracle.softmax(x.numpy()))
    want = torch_cpu.softmax(x)
    if dtype == torch.float16:
        # both are roundings of the same real number up to the library's fp32 error: at most 1 ulp apart
        ulp = _ulp16(got, want)
        assert ulp <= 1
    else:
        assert torch.allclose(got, want, rtol=2e-6, atol=atol)


def test_softmax_invariants(oracle):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(16, 300, generator=g).numpy()
    y = oracle.softmax(x)
    assert np.allclose(y.sum(-1), 1.0, atol=1e-6)
    assert np.allclose(oracle.softmax(x + 3.25), y, rtol=1e-5, atol=1e-9)       # shift invariance
    order = np.argsort(x, -1)
    assert (np.diff(np.take_along_axis(y, order, -1), axis=-1) >= 0).all()     # monotone
    # two-element closed form: softmax([a, b])[0] = 1 / (1 + exp(b - a))
    ab = np.float32([[0.5, -1.25]])
    assert abs(oracle.softmax(ab)[0, 0] - 1.0 / (1.0 + math.exp(-1.75))) < 1e-7


@pytest.mark.parametrize("block", [32, 64, 100])
def test_online_softmax_matches_direct(oracle, block):
    # test_online_softmax.py:21-23: 128x128 fp32; the online recurrence must equal the direct form
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(128, 128, generator=g) * 4).numpy()
    assert np.allclose(oracle.online_softmax_f32(x, block), oracle.softmax(x), rtol=1e-5, atol=1e-8)
    assert torch.allclose(_t(oracle.online_softmax_f32(x, block)), torch_cpu.softmax(_t(x)), atol=1e-5)


# ---------------------------------------------------------------------- norms
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_rms_norm_vs_torch(oracle, dtype):
    # test_rms_norm.py:20-27: 127x513, rand inputs, eps 1e-5
    g = torch.Generator().manual_seed(4)
    x = torch.rand(127, 513, generator=g).to(dtype)
    w = torch.rand(513, generator=g).to(dtype)
    got = _t(oracle.rms_norm(x.numpy(), w.numpy(), 1e-5))
    want = torch_cpu.rms_norm(x, w, 1e-5)
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=2e-6, atol=1e-7)
    else:
        assert _ulp16(got, want) <= 1


def test_rms_norm_closed_form(oracle):
    # constant row c: y = c / sqrt(c^2 + eps) * g ; scaling x by 2 with eps=0 leaves y unchanged
    x = np.full((3, 64), 2.0, np.float32)
    w = np.arange(64, dtype=np.float32)
    y = oracle.rms_norm(x, w, 1e-5)
    assert np.allclose(y, 2.0 / math.sqrt(4.0 + 1e-5) * w, rtol=1e-6)
    g = torch.Generator().manual_seed(5)
    xr = torch.randn(5, 77, generator=g).numpy()
    wr = torch.randn(77, generator=g).numpy()
    assert np.allclose(oracle.rms_norm(2 * xr, wr, 0.0), oracle.rms_norm(xr, wr, 0.0), rtol=1e-6, atol=1e-7)
    assert np.allclose(oracle.rms_norm(xr, None, 0.0), xr / np.sqrt((xr.astype(np.float64) ** 2).mean(-1, keepdims=True)),
                       rtol=1e-6)


@pytest.mark.parametrize("dtype,shape", [(torch.float32, (27, 8192)), (torch.float16, (128, 128)),
                                         (torch.float16, (33, 4096))])
def test_layer_norm_vs_torch(oracle, dtype, shape):
    # test_layer_norm.py:20-32 (27x8192 fp32) and test_layernorm_torch.py:24-31 (128x128 fp16)
    g = torch.Generator().manual_seed(6)
    x = torch.rand(*shape, generator=g).to(dtype)
    w = torch.rand(shape[1], generator=g).to(dtype)
    b = torch.rand(shape[1], generator=g).to(dtype)
    y, mean, rstd = oracle.layer_norm(x.numpy(), w.numpy(), b.numpy(), 1e-5)
    want = torch_cpu.layer_norm(x, w, b, 1e-5)
    if dtype == torch.float32:
        assert torch.allclose(_t(y), want, rtol=1e-5, atol=2e-6)
    else:
        assert _close16(_t(y), want, 1e-6)
    xd = x.double()
    assert np.allclose(mean, xd.mean(-1).numpy(), rtol=1e-6, atol=1e-7)
    assert np.allclose(rstd, (1.0 / torch.sqrt(xd.var(-1, unbiased=False) + 1e-5)).numpy(), rtol=1e-6)


def test_layer_norm_invariants(oracle):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(9, 200, generator=g).numpy()
    y, mean, _ = oracle.layer_norm(x, None, None, 1e-5)
    assert np.allclose(y.mean(-1), 0, atol=1e-6)
    y2, mean2, _ = oracle.layer_norm(x + 10.0, None, None, 1e-5)              # shift invariance
    assert np.allclose(y2, y, atol=2e-5) and np.allclose(mean2, mean + 10.0, atol=1e-5)
    # biased variance: for a row [0, 2] var = 1 (unbiased would be 2)
    yy, _, rstd = oracle.layer_norm(np.float32([[0.0, 2.0]]), None, None, 0.0)
    assert np.allclose(rstd, 1.0) and np.allclose(yy, [[-1.0, 1.0]])


# --------------------------------------------------------------------- matmul
@pytest.mark.parametrize("trans_b", [False, True])
def test_matmul_vs_torch(oracle, trans_b):
    # test_matmul.py:26-28: 1024x64 * 64x512 fp16 (rand); here with fp32 output to compare to fp64 torch
    g = torch.Generator().manual_seed(8)
    a = torch.rand(256, 64, generator=g).half()
    b = torch.rand(*((512, 64) if trans_b else (64, 512)), generator=g).half()
    got = oracle.matmul(a.numpy(), b.numpy(), out_dtype=np.float32, trans_b=trans_b)
    want = a.double() @ (b.double().t() if trans_b else b.double())
    assert np.allclose(got, want.numpy(), rtol=1e-6, atol=1e-6)
    got16 = _t(oracle.matmul(a.numpy(), b.numpy(), trans_b=trans_b))
    assert _ulp16(got16, want.half()) == 0


def test_matmul_closed_forms(oracle):
    g = torch.Generator().manual_seed(9)
    a = torch.randn(48, 32, generator=g).half().numpy()
    eye = np.eye(32, dtype=np.float16)
    assert (oracle.matmul(a, eye) == a).all()                                   # identity
    ones = np.ones((32, 40), np.float16)                                        # dense<1.0> weights: row sums
    assert np.allclose(oracle.matmul(a, ones, out_dtype=np.float32), a.astype(np.float64).sum(-1, keepdims=True))
    twos = np.full((32, 40), 2.0, np.float16)                                   # dense<2.0>
    assert np.allclose(oracle.matmul(a, twos, out_dtype=np.float32), 2 * a.astype(np.float64).sum(-1, keepdims=True))
    onehot = np.zeros((32, 8), np.float16)
    onehot[5, 3] = 1                                                            # picks column 5 of A into column 3
    c = oracle.matmul(a, onehot)
    assert (c[:, 3] == a[:, 5]).all() and (np.delete(c, 3, 1) == 0).all()
    # non-square: a transposed-operand mistake changes the shape-dependent result
    b = torch.randn(32, 24, generator=g).half().numpy()
    assert np.allclose(oracle.matmul(a, b, out_dtype=np.float32), a.astype(np.float64) @ b.astype(np.float64))
    assert np.allclose(oracle.matmul(a, np.ascontiguousarray(b.T), out_dtype=np.float32, trans_b=True),
                       a.astype(np.float64) @ b.astype(np.float64))


def test_matmul_bf16(oracle):
    g = torch.Generator().manual_seed(10)
    a = torch.randn(40, 96, generator=g).bfloat16()
    b = torch.randn(96, 56, generator=g).bfloat16()
    got = oracle.matmul(_bf16_bits(a), _bf16_bits(b), out_dtype="bf16", dtype="bf16")
    want = (a.double() @ b.double()).to(torch.bfloat16)
    assert (got == _bf16_bits(want)).all()


# ---------------------------------------------------------------------- W8A16
def test_dequant_bit_exact(oracle):
    g = torch.Generator().manual_seed(11)
    w = torch.randint(-127, 128, (37, 100), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(37, generator=g)).half()
    got = oracle.dequant_w8(w.numpy(), s.numpy())
    want = w.float() * s.float()[:, None]            # exact int8->f32, one fp32 multiply
    assert (got.view(np.uint32) == want.numpy().view(np.uint32)).all()
    # edges: +-127 and 0 with a power-of-two scale are exact integers / 2^k
    we = np.int8([[127, -127, 0, 1, -1]])
    assert (oracle.dequant_w8(we, np.float16([0.25])) == np.float32([[31.75, -31.75, 0, 0.25, -0.25]])).all()


def test_w8a16_scale_selection_and_indexing(oracle):
    N, K, M = 24, 64, 3
    a = np.zeros((M, K), np.float16)
    a[0, :] = 1.0
    a[1, 7] = 1.0
    a[2, 63] = -2.0
    g = torch.Generator().manual_seed(12)
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).numpy()
    s = np.float16([2.0 ** -(n % 8) for n in range(N)])      # a mis-indexed scale changes a power of two
    c = oracle.matmul_w8a16(a, w, s).astype(np.float64)
    assert np.array_equal(c[0], w.astype(np.int64).sum(1) * s.astype(np.float64))   # exact in fp16 range
    assert np.array_equal(c[1], w[:, 7] * s.astype(np.float64))
    assert np.array_equal(c[2], -2.0 * w[:, 63] * s.astype(np.float64))
    onehot = np.zeros(N, np.float16)
    onehot[5] = 1.0
    c1 = oracle.matmul_w8a16(a, w, onehot)
    assert (np.delete(c1, 5, 1) == 0).all() and c1[1, 5] == w[5, 7]


@pytest.mark.parametrize("M", [1, 16])
def test_w8a16_vs_closed_form(oracle, M):
    g = torch.Generator().manual_seed(13)
    a = torch.randn(M, 512, generator=g).half()
    w = torch.randint(-127, 128, (96, 512), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(96, generator=g)).half()
    got = _t(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    want = (a.double() @ (w.double() * s.double()[:, None]).t())
    assert torch.allclose(got.double(), want, rtol=1e-3, atol=1e-3)
    assert _ulp16(got, want.half()) <= 1


def test_dequant_with_zero_point_and_per_tensor_parameters(oracle):
    # quant.dcast f = (float(q) - zero_point) * scale: integer arithmetic in float64 (exact), then the rounding of
    # the one product to fp32; a dropped or mis-signed zero point, or one taken from the wrong channel, fails
    g = torch.Generator().manual_seed(14)
    w = torch.randint(-128, 128, (21, 50), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(21, generator=g)).half()
    zp = torch.randint(-128, 128, (21,), generator=g, dtype=torch.int8)
    got = oracle.dequant_w8_ex(w.numpy(), s.numpy(), zp.numpy())
    want = ((w.double() - zp.double()[:, None]) * s.double()[:, None]).float()
    assert (got.view(np.uint32) == want.numpy().view(np.uint32)).all()
    # per tensor: index 0 for every channel
    got = oracle.dequant_w8_ex(w.numpy(), s.numpy(), zp.numpy(), per_tensor=True)
    want = ((w.double() - float(zp[0])) * float(s[0])).float()
    assert (got.view(np.uint32) == want.numpy().view(np.uint32)).all()
    # q == zero_point is exactly 0; scale 1 gives the integer difference; no zero point is the symmetric form
    eq = oracle.dequant_w8_ex(np.int8([[5, 5], [-7, -7]]), np.float16([3.0, 2.0]), np.int8([5, -7]))
    assert (eq == 0).all()
    d = oracle.dequant_w8_ex(np.int8([[127, -128]]), np.float16([1.0]), np.int8([-128]))
    assert (d == np.float32([[255.0, 0.0]])).all()
    assert (oracle.dequant_w8_ex(w.numpy(), s.numpy()).view(np.uint32) == oracle.dequant_w8(w.numpy(), s.numpy()).view(np.uint32)).all()


@pytest.mark.parametrize("per_tensor", [False, True])
def test_w8a16_with_zero_point_vs_closed_form(oracle, per_tensor):
    g = torch.Generator().manual_seed(15)
    a = torch.randn(5, 256, generator=g).half()
    w = torch.randint(-128, 128, (40, 256), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(40, generator=g)).half()
    zp = torch.randint(-20, 21, (40,), generator=g, dtype=torch.int8)
    got = _t(oracle.matmul_w8a16_ex(a.numpy(), w.numpy(), s.numpy(), zp.numpy(), per_tensor))
    sd = s.double()[0].expand(40) if per_tensor else s.double()
    zd = zp.double()[0].expand(40) if per_tensor else zp.double()
    want = a.double() @ ((w.double() - zd[:, None]) * sd[:, None]).t()
    assert _ulp16(got, want.half()) <= 1
    # the zero point's share is -zp * s * rowsum(A): a row of ones makes it visible on its own
    ones = np.ones((1, 256), np.float16)
    c = oracle.matmul_w8a16_ex(ones, np.zeros((40, 256), np.int8), np.ones(40, np.float16), zp.numpy(), per_tensor)
    assert np.array_equal(c[0].astype(np.float64), -256.0 * zd.numpy())


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("causal", [False, True])
def test_attention_vs_sdpa(oracle, causal):
    g = torch.Generator().manual_seed(14)
    q, k, v = (torch.randn(2, 3, 96, 32, generator=g) for _ in range(3))
    got = oracle.attention(q.numpy(), k.numpy(), v.numpy(), 0.3, causal)
    want = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=causal, scale=0.3)
    assert np.allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)
    want32 = torch_cpu.attention(q, k, v, 0.3, causal)
    assert np.allclose(got, want32.numpy(), rtol=1e-4, atol=1e-5)


def test_attention_reference_config(oracle):
    # test_flash_attention.py:20-34: Z=H=1, N_CTX=1024, D=64 fp32, rand inputs, scale 0.5, non-causal
    g = torch.Generator().manual_seed(15)
    q, k, v = (torch.rand(1, 1, 1024, 64, generator=g) for _ in range(3))
    got = oracle.attention(q.numpy(), k.numpy(), v.numpy(), 0.5, False)
    want = F.scaled_dot_product_attention(q, k, v, scale=0.5)
    assert torch.allclose(_t(got), want, rtol=1e-5, atol=1e-6)


def test_attention_causal_invariants(oracle):
    g = torch.Generator().manual_seed(16)
    q, k, v = (torch.randn(1, 2, 64, 16, generator=g).numpy() for _ in range(3))
    o = oracle.attention(q, k, v, 0.25, True)
    assert np.allclose(o[:, :, 0, :], v[:, :, 0, :], atol=1e-7)               # row 0 sees only key 0
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 32:, :] = 9.0
    v2[:, :, 32:, :] = -7.0                                                    # later keys do not affect earlier rows
    assert np.array_equal(oracle.attention(q, k2, v2, 0.25, True)[:, :, :32], o[:, :, :32])
    # fp16 in, fp32 out (the HexKL attention fixture's types, hexkl_attention/input.mlir)
    o16 = oracle.attention(q.astype(np.float16), k.astype(np.float16), v.astype(np.float16), 0.25, True,
                           out_dtype=np.float32)
    assert o16.dtype == np.float32 and np.allclose(o16, o, atol=2e-2)


def test_attention_masked_vs_sdpa(oracle):
    # tm_tensor.attention (LowerTmTensor.cpp:70-235): rectangular scores, additive mask with -inf entries
    g = torch.Generator().manual_seed(18)
    B, Sq, Skv, D = 3, 40, 72, 32
    q = torch.randn(B, Sq, D, generator=g)
    k, v = torch.randn(B, Skv, D, generator=g), torch.randn(B, Skv, D, generator=g)
    mask = torch.randn(B, Sq, Skv, generator=g)
    mask[torch.rand(B, Sq, Skv, generator=g) < 0.3] = float("-inf")
    mask[:, :, 0] = 0.0                                                        # no row loses every key
    scale = 1.0 / np.sqrt(D)
    got = oracle.attention_masked(q.numpy(), k.numpy(), v.numpy(), mask.numpy(), scale)
    want = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), attn_mask=mask.double(), scale=scale)
    assert np.allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(got, torch_cpu.attention_masked(q, k, v, mask, scale).numpy(), rtol=1e-4, atol=1e-5)
    # no mask and Sq == Skv: the plain oracle; a causal additive mask: the causal oracle
    q2 = torch.randn(B, Skv, D, generator=g)
    plain = oracle.attention_masked(q2.numpy(), k.numpy(), v.numpy(), None, scale)
    assert np.allclose(plain, oracle.attention(q2.numpy(), k.numpy(), v.numpy(), scale, False), rtol=1e-12, atol=0)
    tri = torch.full((Skv, Skv), float("-inf")).triu(1).expand(B, Skv, Skv).contiguous()
    causal = oracle.attention_masked(q2.numpy(), k.numpy(), v.numpy(), tri.numpy(), scale)
    assert np.allclose(causal, oracle.attention(q2.numpy(), k.numpy(), v.numpy(), scale, True), rtol=1e-12, atol=0)
    # a constant added to a whole mask row changes nothing (shift invariance of the softmax)
    shifted = oracle.attention_masked(q.numpy(), k.numpy(), v.numpy(), (mask + 3.0).numpy(), scale)
    assert np.allclose(shifted, got, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("block_n", [16, 64])
def test_attention_online_recurrence(oracle, block_n):
    g = torch.Generator().manual_seed(17)
    q, k, v = (torch.rand(1, 1, 128, 64, generator=g).numpy() for _ in range(3))
    got = oracle.attention_online_f32(q, k, v, 0.5, block_n)
    want = oracle.attention(q, k, v, 0.5, False)
    assert np.allclose(got, want, rtol=2e-5, atol=1e-6)


# ---- element-wise operators, block sums, rotary embedding ---------------------------------------------------
def test_unary_ops_vs_torch(oracle):
    g = torch.Generator().manual_seed(30)
    x = torch.randn(16384, generator=g, dtype=torch.float64).float() * 3
    xn = x.numpy()
    # test_gelu.py:73-76 (atol 1e-5 in fp32: the kernel's rounded constants differ from torch's in the 7th digit)
    assert np.allclose(oracle.unary("gelu_tanh", xn), F.gelu(x, approximate="tanh").numpy(), atol=1e-5)
    assert np.allclose(oracle.unary("silu", xn), F.silu(x.double()).numpy(), rtol=1e-6, atol=1e-7)   # test_silu.py:69
    pos = torch.rand(1024, generator=g) + 1e-3
    assert np.allclose(oracle.unary("rsqrt", pos.numpy()), torch.rsqrt(pos.double()).numpy(), rtol=1e-6)
    lin = torch.linspace(0, 3.14, 1024)                                          # test_math_ops.py:42
    assert np.allclose(oracle.unary("sin", lin.numpy()), torch.sin(lin.double()).numpy(), atol=1e-7)
    assert np.allclose(oracle.unary("cos", lin.numpy()), torch.cos(lin.double()).numpy(), atol=1e-7)
    assert np.allclose(oracle.unary("exp", xn), torch.exp(x.double()).numpy(), rtol=1e-6)
    # fp16 storage: computed in double, rounded once
    h = x.half()
    want = F.silu(h.double()).half()
    assert np.array_equal(oracle.unary("silu", h.numpy()), want.numpy())
    # closed forms: gelu(0) = 0, silu(0) = 0, gelu(x) -> x for large x and -> 0 for very negative x (no NaN)
    edge = np.array([0.0, 30.0, -30.0, 1e4, -1e4], np.float32)
    assert np.allclose(oracle.unary("gelu_tanh", edge), [0.0, 30.0, 0.0, 1e4, 0.0], atol=1e-6)


def test_binary_ops_and_block_sum(oracle):
    g = torch.Generator().manual_seed(31)
    a, b = torch.rand(5000, generator=g), torch.rand(5000, generator=g) + 0.5
    for name, fn in (("add", torch.add), ("sub", torch.sub), ("mul", torch.mul), ("div", torch.div)):
        assert np.allclose(oracle.binary(name, a.numpy(), b.numpy()), fn(a.double(), b.double()).numpy(), rtol=1e-6)
    x = torch.randn(1024 * 1024, generator=torch.Generator().manual_seed(42))    # test_sum.py:25-27
    assert np.allclose(oracle.block_sum(x.numpy(), x.numel()), torch.sum(x.double()).numpy(), rtol=1e-6, atol=1e-4)
    parts = oracle.block_sum(x.numpy(), 1000)                                    # ragged last program
    assert parts.shape == (1049,)
    assert np.allclose(parts, [c.double().sum().item() for c in torch.split(x, 1000)], rtol=1e-5, atol=1e-5)
    assert np.array_equal(oracle.block_sum(np.arange(12, dtype=np.float32), 4), [6.0, 22.0, 38.0])


def _rope_torch(x, theta):
    """rope_reference_pytorch (test/python/triton/test_rope.py:60-95) in float64."""
    B, L, H, D = x.shape
    idx = torch.arange(D, dtype=torch.float64)
    steps = torch.where(idx % 2 == 0, idx, idx - 1)
    freqs = 1.0 / (theta ** (steps / D))
    ang = torch.arange(L, dtype=torch.float64)[:, None] * freqs[None, :]
    cos, sin = torch.cos(ang).reshape(1, L, 1, D), torch.sin(ang).reshape(1, L, 1, D)
    xd = x.double()
    fwd, bwd = torch.roll(xd, -1, 3), torch.roll(xd, 1, 3)
    even = (torch.arange(D) % 2 == 0).view(1, 1, 1, D)
    return torch.where(even, xd * cos - fwd * sin, bwd * sin + xd * cos)


def test_rope_vs_reference_formula(oracle):
    g = torch.Generator().manual_seed(32)
    x = torch.rand(3, 8, 16, 32, generator=g)                                    # test_rope.py:20-23 shape
    got = oracle.rope(x.numpy(), 10000.0)
    assert np.allclose(got, _rope_torch(x, 10000.0).numpy(), rtol=1e-6, atol=1e-6)
    assert np.array_equal(got[:, 0], x.numpy()[:, 0])                            # position 0: no rotation
    pairs_in = x.numpy().reshape(3, 8, 16, 16, 2)
    pairs_out = got.reshape(3, 8, 16, 16, 2)
    assert np.allclose((pairs_out ** 2).sum(-1), (pairs_in ** 2).sum(-1), rtol=1e-5)   # rotations keep the norm
    x2 = torch.randn(1, 300, 2, 64, generator=g)
    assert np.allclose(oracle.rope(x2.numpy(), 500.0), _rope_torch(x2, 500.0).numpy(), rtol=1e-5, atol=1e-5)


def test_pack_w8_is_the_documented_permutation(oracle):
    # independent statement with reshape / transpose: [T,16,S,4,16] -> [T,S,4,16,16]
    g = torch.Generator().manual_seed(33)
    w = torch.randint(-128, 128, (40, 192), generator=g, dtype=torch.int8).numpy()
    got = oracle.pack_w8(w)
    padded = np.zeros((48, 192), np.int8)
    padded[:40] = w
    want = padded.reshape(3, 16, 3, 4, 16).transpose(0, 2, 3, 1, 4).reshape(-1)
    assert np.array_equal(got, want)
    # every input byte appears exactly once (pure permutation plus zero padding)
    ids = (np.arange(48 * 192, dtype=np.int64) % 251).astype(np.int8).reshape(48, 192)
    assert sorted(oracle.pack_w8(ids).tolist()) == sorted(ids.reshape(-1).tolist())


def test_linear_pins(oracle):
    # (1) against torch's own fused form in fp64; (2) special cases a dropped or mis-indexed operand would fail:
    # zero weights leave bias + residual exactly, a one-hot weight copies a column of A, the bias goes along columns
    g = torch.Generator().manual_seed(21)
    a = torch.randn(24, 40, generator=g).half()
    b = torch.randn(40, 56, generator=g).half()
    bias = torch.randn(56, generator=g).half()
    res = torch.randn(24, 56, generator=g).half()
    got = torch.from_numpy(oracle.linear(a.numpy(), b.numpy(), bias.numpy(), res.numpy()))
    want = torch.addmm(res.double() + bias.double(), a.double(), b.double())
    assert (got.double() - want).abs().max() <= 2e-2 * want.abs().max() / 16
    got_t = torch.from_numpy(oracle.linear(a.numpy(), b.t().contiguous().numpy(), bias.numpy(), res.numpy(), trans_b=True))
    assert torch.equal(got, got_t)
    zero = torch.zeros_like(b)
    only = torch.from_numpy(oracle.linear(a.numpy(), zero.numpy(), bias.numpy(), res.numpy(), out_dtype=np.float32))
    assert torch.equal(only, (res.float() + bias.float()))
    onehot = torch.zeros(40, 56).half()
    onehot[7, 13] = 1
    col = torch.from_numpy(oracle.linear(a.numpy(), onehot.numpy(), bias.numpy(), None, out_dtype=np.float32))
    assert torch.equal(col[:, 13], a[:, 7].float() + bias[13].float())
    assert torch.equal(col[:, 12], bias[12].float().expand(24))
    assert torch.equal(torch.from_numpy(oracle.linear(a.numpy(), b.numpy())),
                       torch.from_numpy(oracle.matmul(a.numpy(), b.numpy())))


def test_add_matmul_softmax_pins(oracle):
    # the reference test's own comparison (test/python/torch-mlir/test_add_matmul_softmax.py:32-60: three 32x32
    # fp32 randn, rtol 1e-5, atol 1e-6) plus what the mathematics fixes: rows sum to 1, y = -x gives the uniform
    # distribution, a shift of every score of a row (z with equal columns added) changes nothing
    g = torch.Generator().manual_seed(22)
    x, y, z = (torch.randn(32, 32, generator=g) for _ in range(3))
    got = torch.from_numpy(oracle.add_matmul_softmax(x.numpy(), y.numpy(), z.numpy()))
    want = torch.softmax(torch.matmul(x + y, z), dim=-1)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)
    assert torch.allclose(got.sum(-1), torch.ones(32), atol=1e-6)
    uniform = torch.from_numpy(oracle.add_matmul_softmax(x.numpy(), (-x).numpy(), z.numpy()))
    assert torch.allclose(uniform, torch.full((32, 32), 1 / 32), atol=1e-7)
    shifted = z + torch.randn(32, 1, generator=g)                    # adds (x + y)[m,:] . c to every score of row m
    got2 = torch.from_numpy(oracle.add_matmul_softmax(x.numpy(), y.numpy(), shifted.numpy()))
    assert torch.allclose(got2, got, rtol=1e-4, atol=1e-6)
    xh, yh, zh = x.half(), y.half(), z.half()
    goth = torch.from_numpy(oracle.add_matmul_softmax(xh.numpy(), yh.numpy(), zh.numpy()))
    wanth = torch.softmax((xh + yh).double() @ zh.double(), dim=-1)
    assert (goth.double() - wanth).abs().max() <= 1e-3
