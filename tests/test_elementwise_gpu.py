"""GPU parity of the element-wise operators, block sums and rotary embedding against the CPU oracle, through the
C ABI, plus the reference tests' own call sites and tolerances.

Tolerances: fp32 within rel-err 1e-5 (+ a small absolute floor) of the oracle's double arithmetic; fp16 / bf16
within one unit in the last place of the oracle's rounded value.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from util import close16, from_np, to_np

pytestmark = pytest.mark.gpu


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _check(got, want, dtype, rtol=1e-5, atol32=1e-6, atol16=1e-6):
    got = got.cpu()
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=rtol, atol=atol32), (got - want).abs().max()
    else:
        assert close16(got, want, max_ulp=1, atol=atol16)


SIZES = [16384, 1, 7, 4099, 1 << 20]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("op", ["gelu_tanh", "silu", "rsqrt", "sin", "cos", "exp"])
@pytest.mark.parametrize("n", SIZES)
def test_unary_parity(hexmi, oracle, op, dtype, n):
    x = torch.randn(n, generator=_gen(0)) * 2
    if op == "rsqrt":
        x = x.abs() + 1e-2
    x = x.to(dtype)
    a, tag = to_np(x)
    want = from_np(oracle.unary(op, a, dtype=tag), dtype)
    got = hexmi.unary(op, x.cuda())
    assert got.dtype == dtype and got.shape == x.shape
    _check(got, want, dtype, atol32=2e-7 if op in ("sin", "cos") else 1e-7, atol16=1e-4 if op in ("sin", "cos") else 1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("n", [16384, 5, 4099, 1 << 20])
def test_binary_parity(hexmi, oracle, op, dtype, n):
    g = _gen(1)
    a = torch.randn(n, generator=g).to(dtype)
    b = (torch.rand(n, generator=g) + 0.5).to(dtype)
    an, tag = to_np(a)
    bn, _ = to_np(b)
    want = from_np(oracle.binary(op, an, bn, dtype=tag), dtype)
    got = hexmi.binary(op, a.cuda(), b.cuda())
    if dtype == torch.float32:
        assert torch.equal(got.cpu(), want)                   # one correctly rounded fp32 operation each
    else:
        _check(got, want, dtype)


def test_unary_misaligned_and_inplace(hexmi, oracle):
    base = torch.randn(4101, generator=_gen(2)).cuda()
    x = base[1:]                                              # 4-byte aligned only
    want = torch.from_numpy(oracle.unary("silu", x.cpu().numpy()))
    assert torch.allclose(hexmi.unary("silu", x).cpu(), want, rtol=1e-5, atol=1e-7)
    out = torch.empty(4100)
    ret = hexmi.unary("silu", x.cpu(), out=out)               # host tensors are staged, out filled in place
    assert ret is out and torch.allclose(out, want, rtol=1e-5, atol=1e-7)
    with pytest.raises(ValueError):
        hexmi.unary("tanh", x)
    assert hexmi.unary("exp", torch.empty(0).cuda()).numel() == 0


def test_gelu_edge_values(hexmi):
    x = torch.tensor([0.0, -0.0, 30.0, -30.0, 1e4, -1e4, float("inf"), float("nan")]).cuda()
    got = hexmi.gelu(x).cpu()
    assert torch.equal(got[:6], torch.tensor([0.0, -0.0, 30.0, -0.0, 1e4, -0.0]))
    assert got[6] == float("inf") and torch.isnan(got[7])


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("num_threads", [1, 4])
def test_reference_gelu_silu_call_sites(hexmi, dtype, num_threads):
    # test_gelu.py:33-76 and test_silu.py:24-70: 16384 elements of rand, atol 1e-5 (fp32) / 1e-2 (fp16)
    x = torch.rand(16384, dtype=dtype)
    out = torch.empty_like(x)
    hexmi.kernels.gelu_kernel[(num_threads,)](x, out, BLOCK_SIZE=16384 // num_threads,
                                              enableMultiThreading=num_threads == 1, enableVTCMTiling=False,
                                              enableConvertToHexagonmem=False, enableHexagonmemCopyToDMA=False)
    assert torch.allclose(out, F.gelu(x, approximate="tanh"), atol=1e-2 if dtype == torch.float16 else 1e-5)
    out2 = torch.empty_like(x)
    hexmi.kernels.silu_kernel[(num_threads,)](x, out2, BLOCK_SIZE=16384 // num_threads, enableMultiThreading=False,
                                              enableVTCMTiling=True, enableConvertToHexagonmem=True,
                                              enableHexagonmemCopyToDMA=True, enableLWP=False)
    assert torch.allclose(out2, F.silu(x), atol=1e-2)
    assert torch.allclose(out2.float(), F.silu(x.float()), atol=1e-3 if dtype == torch.float16 else 1e-6)


def test_reference_math_call_sites(hexmi):
    # test_math_ops.py:41-70, test_rsqrt.py:27-35, test_vec_add_with_scalar.py:26-65, test_vec_div_2d.py:58-68
    X = torch.linspace(0, 3.14, 1024, dtype=torch.float32)
    Y = torch.empty_like(X)
    hexmi.kernels.cos_kernel[(1,)](X, Y, BLOCK_SIZE=1024, enableMultiThreading=True, enableVTCMTiling=True,
                                   enableConvertToHexagonmem=True, enableHexagonmemCopyToDMA=True)
    assert torch.allclose(Y, torch.cos(X), atol=1e-5)
    hexmi.kernels.sin_kernel[(1,)](X, Y, BLOCK_SIZE=1024)
    assert torch.allclose(Y, torch.sin(X), atol=1e-5)
    x = torch.rand(1024)
    out = torch.empty_like(x)
    hexmi.kernels.rsqrt_kernel[(1,)](x, out, BLOCK_SIZE=1024)
    assert torch.allclose(out, torch.rsqrt(x), atol=1e-5)
    a, b = torch.rand(16384, dtype=torch.float16), torch.rand(16384, dtype=torch.float16)
    o = torch.empty_like(a)
    hexmi.kernels.add_kernel_scalar[(4,)](a, b, o, 16384, BLOCK_SIZE=4096, enableVTCMTiling=True)
    assert torch.allclose(o, a + b, atol=1e-2)
    p, q = torch.rand(64, 128), torch.rand(64, 128) + 0.1
    r = torch.empty_like(p)
    hexmi.kernels.div_kernel[(1,)](p, q, r, NUM_ROWS=64, NUM_COLS=128)
    assert torch.allclose(r, p / q, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,block", [(1 << 20, 1 << 20), (100000, 1000), (4099, 4099), (12, 4), (1 << 20, 4096)])
def test_block_sum_parity(hexmi, oracle, dtype, n, block):
    x = torch.randn(n, generator=_gen(42)).to(dtype)
    a, tag = to_np(x)
    want = from_np(oracle.block_sum(a, block, dtype=tag), dtype)
    got = hexmi.block_sum(x.cuda(), block).cpu()
    assert got.shape == want.shape
    # fp32 accumulation of `block` terms: error bound ~ sqrt(block) * eps * sum|x|, well inside these
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=1e-4, atol=2e-6 * block ** 0.5 + 1e-6)
    else:
        assert close16(got, want, max_ulp=1, atol=4e-3 * max(1.0, block ** 0.5 / 64))


@pytest.mark.parametrize("n,block", [(1 << 20, None), (300000, 131072), (1 << 21, 1 << 16), (70001, 70001)])
def test_block_sum_large_fp32_programs(hexmi, n, block):
    # fp32 programs of 2^16 elements and more are summed in two passes (runs of 4096 by many workgroups, then per
    # program): same sums as one pass through the library and as float64 on the CPU, ragged tails included
    x = torch.randn(n, generator=_gen(43))
    got = hexmi.block_sum(x.cuda(), block).cpu()
    b = n if block is None else block
    want = torch.stack([x[i:i + b].double().sum() for i in range(0, n, b)])
    assert got.shape == want.shape and got.dtype == torch.float32
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=2e-6 * b ** 0.5)
    from hexmi import _lib
    xd, one_pass = x.cuda(), torch.empty_like(got).cuda()
    assert _lib.lib().hexmi_block_sum(xd.data_ptr(), one_pass.data_ptr(), n, b, _lib.F32, None) == _lib.OK
    assert torch.allclose(got, one_pass.cpu(), rtol=1e-5, atol=2e-6 * b ** 0.5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_block_sum_workspace_entry(hexmi, dtype):
    # the reference test's own shape through the C ABI: one program over 2^20 elements, summed by the whole chip
    # when the caller passes the scratch the size query asks for; 16-bit inputs keep fp32 partial sums
    from hexmi import _lib
    lib = _lib.lib()
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[dtype]
    n = 1 << 20
    x = torch.randn(n, generator=_gen(44)).to(dtype)
    want = x.double().sum().item()
    xd = x.cuda()
    need = lib.hexmi_block_sum_workspace(n, n, code)
    assert need == (n // 4096) * 4
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.zeros(1, dtype=dtype, device="cuda")
    assert lib.hexmi_block_sum_ws(xd.data_ptr(), out.data_ptr(), n, n, code, ws.data_ptr(), need, None) == _lib.OK
    tol = 1e-2 if dtype == torch.float32 else 0.51 if dtype == torch.float16 else 4.1
    assert abs(out.double().item() - want) <= tol
    # too small a workspace is refused; none at all is the one-pass sum
    assert lib.hexmi_block_sum_ws(xd.data_ptr(), out.data_ptr(), n, n, code, ws.data_ptr(), need - 4, None) == _lib.EINVAL
    assert lib.hexmi_block_sum_ws(xd.data_ptr(), out.data_ptr(), n, n, code, None, 0, None) == _lib.OK
    assert abs(out.double().item() - want) <= tol
    # several programs, ragged last one
    n2, b2 = 300000, 131072
    assert lib.hexmi_block_sum_workspace(n2, b2, code) == ((n2 + 4095) // 4096) * 4
    out3 = torch.zeros(3, dtype=dtype, device="cuda")
    assert lib.hexmi_block_sum_ws(xd.data_ptr(), out3.data_ptr(), n2, b2, code, ws.data_ptr(), need, None) == _lib.OK
    want3 = torch.stack([x[:n2][i:i + b2].double().sum() for i in range(0, n2, b2)])
    assert (out3.double().cpu() - want3).abs().max() <= tol


def test_reference_sum_call_site(hexmi):
    # test_sum.py:22-47: one program over 1024*1024 elements, atol 1e-2
    for dtype in (torch.float16, torch.float32):
        x = torch.randn(1024 * 1024, dtype=dtype, generator=_gen(42))
        output = torch.empty((1), dtype=dtype)
        hexmi.kernels.sum_kernel[1,](x, output, BLOCK_SIZE=1024 * 1024, enableMultiThreading=True,
                                     enableVTCMTiling=True, enableConvertToHexagonmem=True,
                                     enableHexagonmemCopyToDMA=True, enableSplitReduction=True)
        ref = torch.sum(x.double())
        assert abs(output.double().item() - ref.item()) <= (1e-2 if dtype == torch.float32 else 0.51)
    x = torch.arange(12, dtype=torch.float32)
    out = torch.zeros(3)
    hexmi.kernels.sum_kernel[(3,)](x, out, BLOCK_SIZE=4)
    assert torch.equal(out, torch.tensor([6.0, 22.0, 38.0]))


ROPE_SHAPES = [(4, 8, 16, 32), (1, 300, 2, 64), (2, 17, 3, 128), (1, 5, 1, 6), (2, 4096, 4, 128), (3, 2, 40, 16)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", ROPE_SHAPES)
def test_rope_parity(hexmi, oracle, dtype, shape):
    x = torch.randn(*shape, generator=_gen(3)).to(dtype)
    a, tag = to_np(x)
    want = from_np(oracle.rope(a, 10000.0, dtype=tag), dtype)
    got = hexmi.rope(x.cuda(), 10000.0)
    _check(got, want, dtype, rtol=1e-5, atol32=2e-6, atol16=1e-5)
    assert torch.equal(got[:, 0].cpu(), x[:, 0])              # position 0 is the identity


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("num_threads", [1, 4])
def test_reference_rope_call_site(hexmi, dtype, num_threads):
    # test_rope.py:97-240: [BATCH, 8, 16, 32], theta 10000, atol 1e-2 (fp16) / 1e-3 (fp32)
    B, L, H, D = 4, 8, 16, 32
    x = torch.rand(B, L, H, D, dtype=dtype)
    output = torch.empty_like(x)
    hexmi.kernels.rope_kernel[(num_threads,)](
        x, output, BATCH_SIZE=B, BATCH_SIZE_STRIDE=L * H * D, SEQ_LEN=L, SEQ_LEN_STRIDE=H * D, N_HEADS=H,
        N_HEADS_STRIDE=D, N_FEATURES=D, N_FEATURES_STRIDE=1, BLOCK_SIZE=max(B // num_threads, 1), THETA=10000.0,
        enableMultiThreading=num_threads == 1, enableVTCMTiling=num_threads == 1)
    idx = torch.arange(D, dtype=torch.float32)
    steps = torch.where(idx % 2 == 0, idx, idx - 1)
    ang = torch.arange(L, dtype=torch.float32)[:, None] * (1.0 / (10000.0 ** (steps / D)))[None, :]
    cos, sin = torch.cos(ang).reshape(1, L, 1, D), torch.sin(ang).reshape(1, L, 1, D)
    even = (torch.arange(D) % 2 == 0).view(1, 1, 1, D)
    ref = torch.where(even, x * cos - torch.roll(x, -1, 3) * sin, torch.roll(x, 1, 3) * sin + x * cos).to(dtype)
    torch.testing.assert_close(output, ref, atol=1e-2 if dtype == torch.float16 else 1e-3, rtol=0)
    with pytest.raises(ValueError):
        hexmi.rope(torch.zeros(2, 3, 4, 5))
