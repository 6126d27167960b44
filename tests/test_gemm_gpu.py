"""GPU parity of the dense GEMM against the CPU oracle, through the C ABI.

Tolerances. The kernel accumulates in fp32 on the matrix cores; the oracle accumulates in double.
  fp32 output: |got - want| <= 1e-5 * sum_k |a_ik b_kj| (rel-err 1e-5 of the magnitude actually summed; the
    plain rel-err of max|C| is reported by the config-size test and must be <= 1e-5 as well);
  fp16 / bf16 output: within one unit in the last place of the oracle's rounded value, or within 1e-5 of the
    summed magnitude where the value is a cancellation residue. (A flat 2e-2 max-abs is
    also asserted after scaling by 1/sqrt(K), the scale attention-sized outputs have; at |c| ~ 100 one fp16 ulp
    is 0.06, so the raw bound cannot hold for any implementation.)
"""
import math

import numpy as np
import pytest
import torch

from util import close16, from_np, rel_err, to_np

pytestmark = pytest.mark.gpu


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _inputs(M, N, K, dtype, trans_b, seed=0):
    g = _gen(seed)
    a = (2 * torch.rand(M, K, generator=g) - 1).to(dtype)
    b = (2 * torch.rand(*((N, K) if trans_b else (K, N)), generator=g) - 1).to(dtype)
    return a, b


def _oracle_mm(oracle, a, b, out_dtype, trans_b):
    an, tag = to_np(a)
    bn, _ = to_np(b)
    if out_dtype == torch.float32:
        return torch.from_numpy(oracle.matmul(an, bn, out_dtype=np.float32, trans_b=trans_b, dtype=tag))
    od = "bf16" if out_dtype == torch.bfloat16 else np.float16
    return from_np(oracle.matmul(an, bn, out_dtype=od, trans_b=trans_b, dtype=tag), out_dtype)


SHAPES = [
    (1024, 512, 64),      # test_matmul.py:26-28
    (256, 256, 64), (512, 768, 128), (256, 512, 192),
    (100, 72, 64), (300, 264, 128),          # ragged M / N on the tiled path
    (256, 256, 96), (300, 264, 160),         # K % 64 == 32: the four-stage 32-wide-slab kernel
    (384, 256, 320),                         # odd number of 64-wide slabs
    (33, 17, 40), (1, 8, 8), (65, 130, 24), (7, 5, 3),   # any-shape kernel (and, [N,K] weights, the ragged-K one)
    (300, 264, 1000), (130, 136, 72),        # K % 8 == 0 only: the 32-wide-slab kernel with a masked last slab
    (200, 257, 96), (260, 1003, 72),         # ... with an odd N: rows leave through LDS ([N,K]); any-shape ([K,N])
    (300, 1001, 256), (129, 70, 64),         # odd N, whole 64-wide slabs: the paired-slab kernel, element stores
    (130, 136, 2049), (257, 129, 333),       # K % 8 != 0: unaligned rows, the any-shape kernel
]


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_gemm_parity(hexmi, oracle, shape, dtype, trans_b):
    M, N, K = shape
    a, b = _inputs(M, N, K, dtype, trans_b)
    got32 = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32, trans_b=trans_b).cpu()
    want32 = _oracle_mm(oracle, a, b, torch.float32, trans_b)
    bb = b.float().t() if trans_b else b.float()
    mag = a.float().abs() @ bb.abs()
    assert ((got32 - want32).abs() <= 1e-5 * mag + 1e-30).all()
    got = hexmi.matmul(a.cuda(), b.cuda(), trans_b=trans_b).cpu()
    want = _oracle_mm(oracle, a, b, dtype, trans_b)
    # values that are cancellation residues (|c| << sum |a b|) carry the fp32 rounding of the larger partial sums
    assert got.dtype == dtype and close16(got, want, max_ulp=1, atol=1e-5 * float(mag.max()))
    assert ((got.float() - want.float()).abs().max() / math.sqrt(K)) <= 2e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 9, 12, 13, 16, 17, 32, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(64, 8), (100, 64), (4096, 2048), (1000, 2056), (257, 4096), (130, 11008)])
def test_gemm_few_rows_against_transposed_weights(hexmi, oracle, dtype, M, N, K):
    # up to 64 rows with B as [N,K]: the weight-streaming kernels (a wave per output channel up to eight rows, a
    # workgroup per 16 channels on the matrix cores beyond), with and without the epilogue operands, 16-bit and fp32
    # results
    a, b = _inputs(M, N, K, dtype, True, seed=M + N)
    got32 = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32, trans_b=True).cpu()
    want32 = _oracle_mm(oracle, a, b, torch.float32, True)
    mag = a.float().abs() @ b.float().t().abs()
    assert ((got32 - want32).abs() <= 1e-5 * mag + 1e-30).all()
    got = hexmi.matmul(a.cuda(), b.cuda(), trans_b=True).cpu()
    want = _oracle_mm(oracle, a, b, dtype, True)
    assert got.dtype == dtype and close16(got, want, max_ulp=1, atol=1e-5 * float(mag.max()))
    g = _gen(K)
    bias, resid = torch.randn(N, generator=g).to(dtype), torch.randn(M, N, generator=g).to(dtype)
    fused = hexmi.matmul(a.cuda(), b.cuda(), trans_b=True, bias=bias.cuda(), residual=resid.cuda()).cpu()
    ref = (want32.double() + bias.double() + resid.double()).to(dtype)
    assert close16(fused, ref, max_ulp=1, atol=2e-5 * float(mag.max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
@pytest.mark.parametrize("N,K", [(64, 8), (104, 64), (4096, 2048), (1000, 2056), (256, 4096), (136, 11008)])
def test_gemm_few_rows_against_row_major_weights(hexmi, oracle, dtype, M, N, K):
    # a few rows with B as [K,N] (these run on the tiles: a kernel that streams B in 64-byte pieces measured slower)
    a, b = _inputs(M, N, K, dtype, False, seed=M + N)
    got32 = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32).cpu()
    want32 = _oracle_mm(oracle, a, b, torch.float32, False)
    mag = a.float().abs() @ b.float().abs()
    assert ((got32 - want32).abs() <= 1e-5 * mag + 1e-30).all()
    got = hexmi.matmul(a.cuda(), b.cuda()).cpu()
    want = _oracle_mm(oracle, a, b, dtype, False)
    assert got.dtype == dtype and close16(got, want, max_ulp=1, atol=1e-5 * float(mag.max()))
    g = _gen(K)
    bias, resid = torch.randn(N, generator=g).to(dtype), torch.randn(M, N, generator=g).to(dtype)
    fused = hexmi.matmul(a.cuda(), b.cuda(), bias=bias.cuda(), residual=resid.cuda()).cpu()
    ref = (want32.double() + bias.double() + resid.double()).to(dtype)
    assert close16(fused, ref, max_ulp=1, atol=2e-5 * float(mag.max()))


def test_gemm_closed_forms(hexmi):
    g = _gen(1)
    a = torch.randn(256, 128, generator=g).half()
    eye = torch.eye(128).half()
    assert torch.equal(hexmi.matmul(a.cuda(), eye.cuda()).cpu(), a)
    ones = torch.ones(128, 256).half()
    got = hexmi.matmul(a.cuda(), ones.cuda(), out_dtype=torch.float32).cpu()
    assert torch.allclose(got, a.double().sum(-1, keepdim=True).float().expand(256, 256), rtol=1e-5, atol=1e-5)
    onehot = torch.zeros(128, 256).half()
    onehot[5, 200] = 1
    c = hexmi.matmul(a.cuda(), onehot.cuda()).cpu()
    assert torch.equal(c[:, 200], a[:, 5]) and c.abs().sum() == a[:, 5].abs().sum()
    # transposed operand: a row-index / column-index swap in either loader changes this
    b = torch.randn(128, 264, generator=g).half()
    c1 = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32).cpu()
    c2 = hexmi.matmul(a.cuda(), b.t().contiguous().cuda(), out_dtype=torch.float32, trans_b=True).cpu()
    assert torch.equal(c1, c2)


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_large_ragged_tiles(hexmi, dtype, trans_b):
    # enough 256x256 tiles for the large-tile kernel, ragged in M and N, odd slab count; checked on sampled rows
    # against a float64 product of the same rounded inputs
    M, N, K = 2900, 2904, 192
    a, b = _inputs(M, N, K, dtype, trans_b, seed=11)
    got = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32, trans_b=trans_b).cpu()
    rows = torch.cat([torch.arange(0, M, 37), torch.arange(M - 50, M)])
    bb = b.double().t() if trans_b else b.double()
    want = a[rows].double() @ bb
    mag = a[rows].double().abs() @ bb.abs()
    assert ((got[rows].double() - want).abs() <= 1e-5 * mag + 1e-30).all()
    got16 = hexmi.matmul(a.cuda(), b.cuda(), trans_b=trans_b).cpu()
    assert torch.equal(got16, got.to(dtype))          # the 16-bit result is the rounded fp32 result, staged or not


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_odd_width_on_large_tiles(hexmi, dtype):
    # [N,K] weights with an odd N and enough tiles for the 256x256 form (a vocabulary-sized projection): the same
    # kernel as with the weight padded to a multiple of 8 rows, only the way out differs -- bit for bit
    M, N, K = 4096, 8193, 128
    a, b = _inputs(M, N, K, dtype, True, seed=13)
    got = hexmi.matmul(a.cuda(), b.cuda(), trans_b=True)
    b_pad = torch.cat([b, torch.zeros(7, K, dtype=dtype)])
    want = hexmi.matmul(a.cuda(), b_pad.cuda(), trans_b=True)
    assert torch.equal(got, want[:, :N])
    rows = torch.arange(0, M, 97)
    ref = a[rows].double() @ b.double().t()
    assert (got.cpu()[rows].double() - ref).abs().max() <= 2e-2 * math.sqrt(K)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_output_rows_off_the_boundaries(hexmi, dtype):
    # [N,K] weights, whole 64-wide slabs, output rows that start anywhere (odd widths, leading dimensions wider than
    # the rows, a base 2 or 6 bytes into its buffer; C ABI): the staged tile leaves in the aligned 16-byte pieces of
    # each row and its ends by elements. Bit for bit the dense call's values, nothing outside the window written.
    from hexmi import _lib
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    dt = _lib.F16 if dtype == torch.float16 else _lib.BF16
    for M, N, K, pad, lead in ((300, 1001, 256, 0, 0), (300, 1001, 256, 3, 1), (129, 70, 64, 1, 3), (520, 777, 128, 6, 0),
                               (4096, 2049, 128, 0, 1), (64, 5, 64, 2, 1), (257, 263, 192, 4, 3)):
        a, b = _inputs(M, N, K, dtype, True, seed=M + N + pad)
        ldc = N + pad
        c_buf = torch.full((M * ldc + lead + 9,), 7.0, dtype=dtype, device="cuda")
        ad, bd = a.cuda(), b.cuda()
        rc = L.hexmi_gemm(M, N, K, ad.data_ptr(), K, bd.data_ptr(), K, c_buf.data_ptr() + 2 * lead, ldc, dt, dt, 1, st)
        assert rc == 0
        b_pad = torch.cat([b, torch.zeros((-N) % 8, K, dtype=dtype)])
        want = hexmi.matmul(ad, b_pad.cuda(), trans_b=True)[:, :N]
        c = c_buf[lead:lead + M * ldc].view(M, ldc)
        assert torch.equal(c[:, :N], want), (M, N, K, pad, lead)
        assert (c_buf[:lead] == 7.0).all() and (c[:, N:] == 7.0).all() and (c_buf[lead + M * ldc:] == 7.0).all()


def test_gemm_unaligned_views(hexmi):
    # operands and result that start 2 bytes into their buffers, odd leading dimensions (C ABI only): the any-shape
    # kernel; nothing outside the result's window is written
    from hexmi import _lib
    L = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    g = _gen(14)
    for trans_b in (0, 1):
        for M, N, K in ((200, 136, 264), (130, 77, 100), (64, 64, 64)):
            lda, ldb, ldc = K + 3, (K if trans_b else N) + 5, N + 1
            a_buf = (2 * torch.rand(M * lda + 1, generator=g) - 1).half().cuda()
            b_buf = (2 * torch.rand((N if trans_b else K) * ldb + 1, generator=g) - 1).half().cuda()
            c_buf = torch.full((M * ldc + 1,), 7.0, dtype=torch.float16, device="cuda")
            rc = L.hexmi_gemm(M, N, K, a_buf.data_ptr() + 2, lda, b_buf.data_ptr() + 2, ldb, c_buf.data_ptr() + 2, ldc,
                              1, 1, trans_b, st)
            assert rc == 0
            a = a_buf[1:].view(M, lda)[:, :K].contiguous()
            b = b_buf[1:].view(-1, ldb)[:, :(K if trans_b else N)].contiguous()
            want = hexmi.matmul(a, b, trans_b=bool(trans_b))
            c = c_buf[1:].view(M, ldc)
            assert close16(c[:, :N].contiguous(), want, max_ulp=1, atol=1e-4)
            assert float(c_buf[0]) == 7.0 and (c[:, N:] == 7.0).all()


def test_gemm_strided_operands(hexmi):
    # leading dimensions larger than the rows (C ABI only): same arithmetic as the dense call, bit for bit; ldc % 8 != 0
    # takes the direct (unstaged) 16-bit stores
    from hexmi import _lib
    L = _lib.lib()
    M, N, K = 300, 264, 128
    lda, ldb, ldc = K + 8, N + 16, N + 4
    g = _gen(12)
    a_big = (2 * torch.rand(M, lda, generator=g) - 1).half().cuda()
    b_big = (2 * torch.rand(K, ldb, generator=g) - 1).half().cuda()
    c_big = torch.full((M, ldc), 7.0, dtype=torch.float16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    rc = L.hexmi_gemm(M, N, K, a_big.data_ptr(), lda, b_big.data_ptr(), ldb, c_big.data_ptr(), ldc, 1, 1, 0, st)
    assert rc == 0
    dense = hexmi.matmul(a_big[:, :K].contiguous(), b_big[:, :N].contiguous())
    assert torch.equal(c_big[:, :N], dense)
    assert (c_big[:, N:] == 7.0).all()                # nothing written past the N columns


def test_hexkl_entry_point(hexmi, oracle):
    # hexmi_matmul_f16f16_f32(n_row, n_col, n_inner, out, act, w): the fixture's sizes
    # (test/python/mlir/hexkl_linalg_matmul/wrapper.cpp:31-33: N=1024, K=64, M=512) and its MAX_DIFF 1e-2
    from hexmi import _lib
    g = _gen(2)
    act = (torch.randn(1024, 64, generator=g) * 0.5).half()
    w = (torch.randn(64, 512, generator=g) * 0.5).half()
    out = torch.empty(1024, 512, device="cuda")
    ad, wd = act.cuda(), w.cuda()
    rc = _lib.lib().hexmi_matmul_f16f16_f32(1024, 512, 64, out.data_ptr(), ad.data_ptr(), wd.data_ptr(),
                                            torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    want = torch.from_numpy(oracle.matmul(act.numpy(), w.numpy(), out_dtype=np.float32))
    assert (out.cpu() - want).abs().max() < 1e-2
    assert rel_err(out, want) <= 1e-5


def test_reference_matmul_call_site(hexmi, oracle):
    # test_matmul.py:72-91: host tensors, C zero-initialised and filled in place, atol 2e-1
    g = _gen(3)
    A = torch.rand((1024, 64), generator=g).half()
    B = torch.rand((64, 512), generator=g).half()
    C = torch.zeros((1024, 512), dtype=torch.float16)
    hexmi.kernels.matmul[(1,)](A, B, C, 1024, 512, 64, enableMultiThreading=True, enableVTCMTiling=True,
                               enableConvertToHexagonmem=True, enableHexagonmemCopyToDMA=True)
    want = from_np(oracle.matmul(A.numpy(), B.numpy()), torch.float16)
    assert torch.allclose(C, want, atol=2e-1) and close16(C, want, 1, atol=1e-4)
    # matmul_hexkl.md:100-111: fp32 C, rtol 1e-2
    C32 = torch.zeros((1024, 512), dtype=torch.float32)
    hexmi.kernels.matmul_hexkl[(1,)](A, B, C32, 1024, 512, 64, enableHexKL=True)
    assert torch.allclose(C32, torch.from_numpy(oracle.matmul(A.numpy(), B.numpy(), out_dtype=np.float32)), rtol=1e-5)


def test_macro_matmul_shapes(hexmi, oracle):
    # test_hexkl_macro_matmul.py:31-68: 1024^3 and x[1024,512] @ W[256,512].T, randn seed 42, rtol/atol 1e-2
    torch.manual_seed(42)
    x = torch.randn(512, 1024).half()
    w = torch.randn(1024, 1024).half()
    got = hexmi.matmul(x.cuda(), w.cuda()).cpu()
    assert close16(got, from_np(oracle.matmul(x.numpy(), w.numpy()), torch.float16), 1, atol=1e-4)
    x2 = torch.randn(1024, 512).half()
    w2 = torch.randn(256, 512).half()
    got2 = hexmi.matmul(x2.cuda(), w2.cuda(), trans_b=True).cpu()
    want2 = from_np(oracle.matmul(x2.numpy(), w2.numpy(), trans_b=True), torch.float16)
    assert close16(got2, want2, 1, atol=1e-4) and torch.allclose(got2.float(), want2.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype,size", [(torch.float16, 4096), (torch.bfloat16, 8192)])
def test_gemm_config_sizes(hexmi, oracle, dtype, size):
    """Measured configurations. The oracle is run on a deterministic subset of rows (every 61st row, all
    columns); the full result is covered by a size-independent property: linearity in A,
    (A + A') B == A B + A' B exactly in fp32 output when A' is a row permutation of A scaled by 0 or 1 --
    here checked as: C computed from a row-shuffled A equals the row-shuffled C, bit for bit."""
    from hexmi.workloads import gemm_inputs
    inp = gemm_inputs(size, size, size, dtype)
    a, b = inp["a"], inp["b"]
    ad, bd = a.cuda(), b.cuda()
    c = hexmi.matmul(ad, bd)
    c32 = hexmi.matmul(ad, bd, out_dtype=torch.float32)
    rows = torch.arange(0, size, 61)
    an, tag = to_np(a[rows])
    bn, _ = to_np(b)
    want32 = torch.from_numpy(oracle.matmul(an, bn, out_dtype=np.float32, dtype=tag))
    got32 = c32[rows.cuda()].cpu()
    assert rel_err(got32, want32) <= 1e-5
    od = "bf16" if dtype == torch.bfloat16 else np.float16
    want = from_np(oracle.matmul(an, bn, out_dtype=od, dtype=tag), dtype)
    assert close16(c[rows.cuda()].cpu(), want, 1, atol=1e-4)
    perm = torch.randperm(size, generator=_gen(7)).cuda()
    c_perm = hexmi.matmul(ad[perm].contiguous(), bd)
    assert torch.equal(c_perm, c[perm])
    # the same product through the transposed-weight loader must agree exactly (same fp32 sums, same order in k)
    c_t = hexmi.matmul(ad, bd.t().contiguous(), trans_b=True)
    assert torch.equal(c_t, c)


def test_gemm_empty_inner_dimension_is_zero(hexmi):
    # a product over K = 0 is all zeros (torch.matmul gives the same), for every output type, with a leading dimension
    for dt, odt in ((torch.float16, torch.float16), (torch.bfloat16, torch.float32), (torch.float32, torch.float32)):
        buf = torch.full((5, 12), 3.0, dtype=odt, device="cuda")
        out = buf[:, :7]
        from hexmi import _lib
        code = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}
        rc = _lib.lib().hexmi_gemm(5, 7, 0, None, 0, None, 7, out.data_ptr(), 12, code[dt], code[odt], 0, None)
        assert rc == _lib.OK
        torch.cuda.synchronize()
        assert torch.equal(buf[:, :7].cpu(), torch.zeros(5, 7, dtype=odt))
        assert torch.equal(buf[:, 7:].cpu(), torch.full((5, 5), 3.0, dtype=odt))       # past N: untouched
    assert hexmi.matmul(torch.zeros(4, 0, dtype=torch.float16, device="cuda"),
                        torch.zeros(0, 8, dtype=torch.float16, device="cuda")).abs().sum().item() == 0


def test_gemm_argument_errors(hexmi):
    from hexmi import _lib
    a = torch.zeros(8, 8, device="cuda", dtype=torch.float16)
    lib = _lib.lib()
    assert lib.hexmi_gemm(8, 8, 8, a.data_ptr(), 4, a.data_ptr(), 8, a.data_ptr(), 8, _lib.F16, _lib.F16, 0, None) == _lib.EINVAL
    assert lib.hexmi_gemm(8, 8, 8, a.data_ptr(), 8, a.data_ptr(), 8, a.data_ptr(), 8, _lib.F32, _lib.F16, 0, None) == _lib.ENOTSUP
    assert lib.hexmi_gemm(8, 8, 8, a.data_ptr(), 8, a.data_ptr(), 8, a.data_ptr(), 8, _lib.F16, _lib.BF16, 0, None) == _lib.ENOTSUP
    with pytest.raises(TypeError):
        hexmi.matmul(torch.zeros(4, 4, device="cuda", dtype=torch.float64), torch.zeros(4, 4, device="cuda", dtype=torch.float64))
    with pytest.raises(ValueError):
        hexmi.matmul(a, torch.zeros(4, 4, device="cuda", dtype=torch.float16))


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("shape", [(32, 32, 32), (1, 1, 1), (65, 130, 17), (200, 77, 300), (512, 512, 512),
                                   # K % 32 == 0 (and N % 4 == 0 for [K,N] operands): the matrix-core kernel; ragged
                                   # tiles on both sides, fewer rows than a fragment, several slabs, odd slab counts
                                   (128, 128, 32), (5, 4, 64), (300, 264, 160), (129, 1028, 96), (1000, 520, 1024),
                                   (2048, 384, 224), (64, 132, 4096)])
def test_matmul_fp32(hexmi, oracle, shape, trans_b):
    M, N, K = shape
    g = torch.Generator().manual_seed(40)
    a = torch.randn(M, K, generator=g)
    b = torch.randn(N, K, generator=g) if trans_b else torch.randn(K, N, generator=g)
    got = hexmi.matmul(a.cuda(), b.cuda(), trans_b=trans_b).cpu()
    want = a.double() @ (b.double().t() if trans_b else b.double())
    assert got.dtype == torch.float32
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-5 * (K ** 0.5))
    with pytest.raises(TypeError):
        hexmi.matmul(a.cuda(), b.cuda(), trans_b=trans_b, out_dtype=torch.float16)


@pytest.mark.parametrize("trans_b", [False, True])
def test_matmul_fp32_strided_and_exact(hexmi, trans_b):
    # operands that are views into wider buffers (leading dimensions larger than the rows), an output view, and
    # small-integer operands whose products and sums are exact in fp32: the result must be exact, whatever the order
    M, N, K = 200, 136, 96
    g = torch.Generator().manual_seed(45)
    abuf = torch.randint(-8, 9, (M, K + 32), generator=g).float().cuda()
    bbuf = (torch.randint(-8, 9, (N, K + 64), generator=g) if trans_b else torch.randint(-8, 9, (K, N + 24), generator=g)).float().cuda()
    cbuf = torch.full((M, N + 8), -1.0, device="cuda")
    a, b, c = abuf[:, :K], (bbuf[:, :K] if trans_b else bbuf[:, :N]), cbuf[:, :N]
    lib, st = hexmi.lib(), torch.cuda.current_stream().cuda_stream
    from hexmi import _lib
    rc = lib.hexmi_gemm(M, N, K, a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), c.data_ptr(), c.stride(0),
                        _lib.F32, _lib.F32, int(trans_b), st)
    assert rc == 0
    torch.cuda.synchronize()
    want = a.double().cpu() @ (b.double().cpu().t() if trans_b else b.double().cpu())
    assert torch.equal(c.cpu().double(), want)
    assert (cbuf[:, N:] == -1.0).all()                       # nothing written past the N columns


def test_add_matmul_softmax_reference_graph(hexmi):
    # test/python/torch-mlir/test_add_matmul_softmax.py:32-60: three 32x32 fp32 randn, rtol 1e-5, atol 1e-6
    g = torch.Generator().manual_seed(41)
    x, y, z = (torch.randn(32, 32, generator=g) for _ in range(3))
    got = hexmi.add_matmul_softmax(x, y, z)
    want = torch.nn.functional.softmax(torch.matmul(x + y, z), dim=-1)
    assert got.device.type == "cuda"
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-6)
    # fp16 operands run the matrix-core GEMM
    got16 = hexmi.add_matmul_softmax(x.half(), y.half(), z.half()).cpu()
    want16 = torch.nn.functional.softmax(torch.matmul((x.half() + y.half()).float(), z.half().float()), dim=-1)
    assert torch.allclose(got16.float(), want16, atol=2e-2)


# ---- hexmi_gemm_ex: bias and residual in the GEMM epilogue ------------------------------------------------------
def _linear_ref(a, b, bias, resid, trans_b):
    c = a.double() @ (b.double().T if trans_b else b.double())
    if bias is not None:
        c = c + bias.double()
    if resid is not None:
        c = c + resid.double()
    return c


@pytest.mark.parametrize("dtype,out_dtype", [(torch.float16, torch.float16), (torch.bfloat16, torch.bfloat16),
                                             (torch.float16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("shape", [(512, 2304, 768), (512, 768, 3072),      # GPT-2 small layers (64-k tiled kernel)
                                   (256, 256, 96),                           # 32-k tiled kernel
                                   (100, 72, 40), (33, 50, 17),              # any-shape kernel (ragged, unaligned)
                                   (260, 1003, 72), (130, 136, 1000),        # ragged-K kernel: rows through LDS / runs
                                   (1024, 1024, 1024)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gemm_ex_bias_and_residual(hexmi, dtype, out_dtype, shape, trans_b):
    M, N, K = shape
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K + trans_b)
    a = (torch.randn(M, K, generator=g) * 0.5).to(dtype)
    b = (torch.randn((N, K) if trans_b else (K, N), generator=g) * 0.5).to(dtype)
    bias = torch.randn(N, generator=g).to(out_dtype)
    resid = torch.randn(M, N, generator=g).to(out_dtype)
    tol = {torch.float16: 2e-2, torch.bfloat16: 1.5e-1, torch.float32: 2e-3 if dtype != torch.float32 else 2e-4}[out_dtype]
    for use_bias, use_resid in ((True, True), (True, False), (False, True)):
        got = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=out_dtype, trans_b=trans_b,
                           bias=bias.cuda() if use_bias else None, residual=resid.cuda() if use_resid else None)
        want = _linear_ref(a, b, bias if use_bias else None, resid if use_resid else None, trans_b)
        err = (got.cpu().double() - want).abs().max().item()
        assert err <= tol * max(1.0, want.abs().max().item() / 16), (use_bias, use_resid, err)


def test_gemm_ex_rounds_once(hexmi):
    # fp16: A B + bias + residual rounded once from fp32 == the correctly rounded fp64 result on all but ties; the
    # separate kernels (round the product, round the sum, round again) are measurably further away.
    g = torch.Generator().manual_seed(11)
    M, N, K = 256, 512, 256
    a = torch.randn(M, K, generator=g).half()
    b = torch.randn(K, N, generator=g).half()
    bias = torch.randn(N, generator=g).half()
    resid = torch.randn(M, N, generator=g).half()
    want = _linear_ref(a, b, bias, resid, False)
    fused = hexmi.matmul(a.cuda(), b.cuda(), bias=bias.cuda(), residual=resid.cuda()).cpu().double()
    parts = hexmi.binary("add", hexmi.binary("add", hexmi.matmul(a.cuda(), b.cuda()),
                                             bias.cuda().expand(M, N).contiguous()), resid.cuda()).cpu().double()
    e_fused = (fused - want).abs().mean().item()
    e_parts = (parts - want).abs().mean().item()
    assert e_fused < e_parts
    assert (fused - want.half().double()).abs().max().item() <= 2 * torch.finfo(torch.float16).eps * want.abs().max().item()


# one shape per kernel that takes a residual: paired 64-k slabs, 32-k slabs (K % 64 != 0), the any-shape kernel
# (odd N), the fp32 matrix-core kernel and the fp32 vector-ALU kernel (K % 32 != 0)
@pytest.mark.parametrize("dtype,M,N,K", [(torch.float16, 384, 768, 768), (torch.float16, 256, 512, 96),
                                         (torch.bfloat16, 200, 333, 64), (torch.float32, 256, 512, 128),
                                         (torch.float32, 130, 77, 50)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gemm_ex_residual_may_alias_output(hexmi, dtype, M, N, K, trans_b):
    g = torch.Generator().manual_seed(12)
    a = (torch.randn(M, K, generator=g) * 0.1).to(dtype).cuda()
    b = (torch.randn(*((N, K) if trans_b else (K, N)), generator=g) * 0.1).to(dtype).cuda()
    x = torch.randn(M, N, generator=g).to(dtype).cuda()
    want = hexmi.matmul(a, b, residual=x, trans_b=trans_b)
    acc = x.clone()
    hexmi.matmul(a, b, residual=acc, out=acc, trans_b=trans_b)      # x += a @ b, in place
    assert torch.equal(acc, want)


def test_gemm_ex_strided_residual_and_bad_arguments(hexmi):
    from hexmi import _lib
    lib = _lib.lib()
    g = torch.Generator().manual_seed(13)
    M, N, K = 128, 256, 128
    a = torch.randn(M, K, generator=g).half().cuda()
    b = torch.randn(K, N, generator=g).half().cuda()
    wide = torch.randn(M, N + 64, generator=g).half().cuda()       # residual with a leading dimension of N + 64
    c = torch.empty(M, N, dtype=torch.float16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    st = lib.hexmi_gemm_ex(M, N, K, a.data_ptr(), K, b.data_ptr(), N, c.data_ptr(), N, None, wide.data_ptr(), N + 64,
                           _lib.F16, _lib.F16, 0, s)
    assert st == 0
    want = _linear_ref(a.cpu(), b.cpu(), None, wide[:, :N].cpu(), False)
    assert (c.cpu().double() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item() / 16)
    # a residual narrower than the result is refused
    assert lib.hexmi_gemm_ex(M, N, K, a.data_ptr(), K, b.data_ptr(), N, c.data_ptr(), N, None, wide.data_ptr(), N - 8,
                             _lib.F16, _lib.F16, 0, s) == _lib.EINVAL
    with pytest.raises(ValueError):
        hexmi.matmul(a, b, bias=torch.zeros(N + 1, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError):
        hexmi.matmul(a, b, residual=torch.zeros(M, N, dtype=torch.float32, device="cuda"))


# ---- hexmi_add_matmul_softmax: the fused graph in one launch ----------------------------------------------------
def _ams_ref(x, y, z):
    total = (x + y)                                                  # torch.add rounds the sum to the dtype
    return torch.softmax(total.double() @ z.double(), dim=-1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(32, 32, 32),                     # test_add_matmul_softmax.py:32-60
                                   (1, 1, 1), (7, 5, 3), (100, 130, 70), (33, 257, 100), (64, 512, 48),
                                   (50, 1000, 37), (96, 1024, 64), (512, 768, 768)])
def test_add_matmul_softmax_one_launch(hexmi, dtype, shape):
    M, N, K = shape
    g = torch.Generator().manual_seed(M + N * 5 + K * 11)
    x = torch.randn(M, K, generator=g).to(dtype)
    y = torch.randn(M, K, generator=g).to(dtype)
    z = (torch.randn(K, N, generator=g) * (1.0 if K <= 64 else 0.2)).to(dtype)
    got = hexmi.add_matmul_softmax(x.cuda(), y.cuda(), z.cuda(), fused=True).cpu()
    want = _ams_ref(x, y, z)
    assert got.dtype == dtype and got.shape == (M, N)
    if dtype == torch.float32:
        # the reference test's own bounds at its size; longer fp32 sums carry their rounding into the exponent
        torch.testing.assert_close(got.double(), want, rtol=1e-5 if K <= 64 else 2e-4, atol=1e-6)
    else:
        eps = torch.finfo(dtype).eps
        torch.testing.assert_close(got.double(), want, rtol=2 * eps, atol=eps * 0.25)
    sums = got.double().sum(-1)
    assert (sums - 1).abs().max().item() <= (1e-5 if dtype == torch.float32 else N ** 0.5 * torch.finfo(dtype).eps)
    # the three-launch route agrees (it rounds the product to the dtype before the softmax, so only to that rounding)
    three = hexmi.add_matmul_softmax(x.cuda(), y.cuda(), z.cuda(), fused=False).cpu()
    tol = 1e-5 if dtype == torch.float32 else 0.02 if dtype == torch.float16 else 0.15
    assert (three.double() - got.double()).abs().max().item() <= tol


def test_add_matmul_softmax_limits_and_layouts(hexmi):
    from hexmi import _lib
    lib = _lib.lib()
    assert lib.hexmi_add_matmul_softmax_max_n() == 1024
    g = torch.Generator().manual_seed(3)
    M, N, K = 40, 96, 24
    s = torch.cuda.current_stream().cuda_stream
    # leading dimensions wider than the rows, output at an odd element offset (no 4-element runs)
    xw = torch.randn(M, K + 3, generator=g).cuda()
    yw = torch.randn(M, K + 5, generator=g).cuda()
    zw = torch.randn(K, N + 7, generator=g).cuda()
    ow = torch.full((M * (N + 1) + 1,), -7.0, device="cuda")
    st = lib.hexmi_add_matmul_softmax(M, N, K, xw.data_ptr(), K + 3, yw.data_ptr(), K + 5, zw.data_ptr(), N + 7,
                                      ow.data_ptr() + 4, N + 1, _lib.F32, s)
    assert st == 0
    got = ow[1:].reshape(M, N + 1).cpu()
    want = _ams_ref(xw[:, :K].cpu(), yw[:, :K].cpu(), zw[:, :N].cpu())
    torch.testing.assert_close(got[:, :N].double(), want, rtol=1e-5, atol=1e-6)
    assert (got[:, N] == -7.0).all() and ow[0].item() == -7.0       # nothing written outside the result
    # too wide, and nonsense sizes
    big = torch.zeros(8, 1025, device="cuda")
    assert lib.hexmi_add_matmul_softmax(8, 1025, 8, big.data_ptr(), 8, big.data_ptr(), 8, big.data_ptr(), 1025,
                                        big.data_ptr(), 1025, _lib.F32, s) == _lib.ETOOBIG
    assert lib.hexmi_add_matmul_softmax(8, 16, 8, big.data_ptr(), 4, big.data_ptr(), 8, big.data_ptr(), 16,
                                        big.data_ptr(), 16, _lib.F32, s) == _lib.EINVAL
    assert lib.hexmi_add_matmul_softmax(0, 16, 8, None, 8, None, 8, None, 16, None, 16, _lib.F32, s) == 0
    # K == 0: every score is an empty sum, every row uniform
    out = torch.empty(5, 10, device="cuda")
    assert lib.hexmi_add_matmul_softmax(5, 10, 0, None, 0, None, 0, None, 10, out.data_ptr(), 10, _lib.F32, s) == 0
    torch.testing.assert_close(out.cpu(), torch.full((5, 10), 0.1))
    with pytest.raises(ValueError):
        hexmi.add_matmul_softmax(big, big, torch.zeros(1025, 2048, device="cuda"), fused=True)


# ---- hexmi_transpose16: one-time weight re-layout ----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 1), (3, 70), (64, 64), (65, 129), (768, 3072), (1000, 37), (4096, 4096)])
def test_pack_weight_is_the_transpose(hexmi, dtype, shape):
    g = torch.Generator().manual_seed(shape[0] * 3 + shape[1])
    w = torch.randn(*shape, generator=g).to(dtype)
    w[0, 0] = float("inf")                                          # bit patterns are moved, whatever they are
    got = hexmi.pack_weight(w.cuda())
    assert got.shape == (shape[1], shape[0]) and got.dtype == dtype and got.is_contiguous()
    assert torch.equal(got.cpu().view(torch.int16), w.t().contiguous().view(torch.int16))


def test_packed_weight_product_is_the_same_product(hexmi):
    # A . B and A . pack(B)^T multiply the same numbers: equal to the last bit in the fp32-output mode
    g = torch.Generator().manual_seed(5)
    a = torch.randn(256, 512, generator=g).half().cuda()
    b = torch.randn(512, 384, generator=g).half().cuda()
    bt = hexmi.pack_weight(b)
    c1 = hexmi.matmul(a, b, out_dtype=torch.float32)
    c2 = hexmi.matmul(a, bt, out_dtype=torch.float32, trans_b=True)
    assert torch.equal(c1, c2)


def test_transpose16_strides_and_bad_arguments(hexmi):
    from hexmi import _lib
    lib = _lib.lib()
    s = torch.cuda.current_stream().cuda_stream
    src = torch.arange(20 * 12, dtype=torch.int16, device="cuda").reshape(20, 12)        # rows 20, ld 12, cols 10 used
    dst = torch.full((10, 24), -1, dtype=torch.int16, device="cuda")
    assert lib.hexmi_transpose16(20, 10, src.data_ptr(), 12, dst.data_ptr(), 24, s) == 0
    assert torch.equal(dst[:, :20].cpu(), src[:, :10].t().cpu())
    assert (dst[:, 20:] == -1).all()
    assert lib.hexmi_transpose16(20, 10, src.data_ptr(), 8, dst.data_ptr(), 24, s) == _lib.EINVAL
    assert lib.hexmi_transpose16(20, 10, src.data_ptr(), 12, dst.data_ptr(), 16, s) == _lib.EINVAL
    assert lib.hexmi_transpose16(0, 10, None, 12, None, 24, s) == 0
    with pytest.raises(TypeError):
        hexmi.pack_weight(torch.zeros(4, 4, device="cuda"))


def test_gemm_ex_and_fused_graph_against_the_oracle(hexmi, oracle):
    # the C oracle's product with its numpy epilogue / softmax (oracle.linear, oracle.add_matmul_softmax), fp16 and fp32
    g = torch.Generator().manual_seed(31)
    a = torch.randn(192, 320, generator=g).half()
    b = (torch.randn(320, 136, generator=g) * 0.2).half()
    bias = torch.randn(136, generator=g).half()
    res = torch.randn(192, 136, generator=g).half()
    got = hexmi.matmul(a.cuda(), b.cuda(), bias=bias.cuda(), residual=res.cuda()).cpu()
    want = torch.from_numpy(oracle.linear(a.numpy(), b.numpy(), bias.numpy(), res.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)
    got32 = hexmi.matmul(a.cuda(), b.cuda(), out_dtype=torch.float32, bias=bias.float().cuda(),
                         residual=res.float().cuda()).cpu()
    want32 = torch.from_numpy(oracle.linear(a.numpy(), b.numpy(), bias.float().numpy(), res.float().numpy(),
                                            out_dtype=np.float32))
    assert torch.allclose(got32, want32, rtol=1e-5, atol=1e-4)
    for dtype in (torch.float32, torch.float16):
        x, y = (torch.randn(70, 48, generator=g).to(dtype) for _ in range(2))
        z = torch.randn(48, 200, generator=g).to(dtype)
        gf = hexmi.add_matmul_softmax(x.cuda(), y.cuda(), z.cuda(), fused=True).cpu()
        wf = torch.from_numpy(oracle.add_matmul_softmax(x.numpy(), y.numpy(), z.numpy()))
        if dtype == torch.float32:
            assert torch.allclose(gf, wf, rtol=1e-5, atol=1e-6)
        else:
            assert close16(gf, wf, max_ulp=1, atol=1e-5)
