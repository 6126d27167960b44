"""GPU parity of flash-attention forward against the brute-force CPU oracle, through the C ABI.

Tolerance: fp16 / bf16 inputs: max-abs <= 2e-2 (outputs are convex combinations of V rows, |o| <~ 4; the
probabilities are rounded to the 16-bit input type before P V as in the reference's linalg form,
test/python/mlir/hexkl_attention/input.mlir:140-145); fp32 inputs: rel-err 1e-5.
"""
import math

import numpy as np
import pytest
import torch

from util import from_np, rel_err, to_np

pytestmark = pytest.mark.gpu


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _qkv(Z, H, S, D, dtype, seed=0, rand=False):
    g = _gen(seed)
    f = torch.rand if rand else torch.randn
    return tuple(f(Z, H, S, D, generator=g).to(dtype) for _ in range(3))


def _oracle(oracle, q, k, v, scale, causal, out_dtype=None):
    qn, tag = to_np(q)
    kn, _ = to_np(k)
    vn, _ = to_np(v)
    o = oracle.attention(qn, kn, vn, scale, causal, out_dtype=np.float32, dtype=tag)
    return torch.from_numpy(o)


CASES = [(1, 1, 1024, 64), (2, 3, 256, 128), (1, 2, 128, 128), (1, 2, 64, 64), (1, 1, 200, 128), (2, 1, 77, 64),
         (1, 1, 1, 128), (1, 3, 129, 128), (1, 1, 640, 128)]


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_attention_parity_half(hexmi, oracle, case, dtype, causal):
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, dtype)
    scale = 1.0 / math.sqrt(D)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal).cpu()
    want = _oracle(oracle, q, k, v, scale, causal)
    assert got.dtype == dtype
    tol = 2e-2 if dtype == torch.float16 else 4e-2
    assert (got.float() - want).abs().max() <= tol
    got32 = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    assert (got32 - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [(1, 2, 300, 80), (2, 1, 129, 96), (1, 3, 64, 32), (1, 1, 513, 8), (2, 8, 200, 48),
                                  (1, 1, 1000, 120), (1, 2, 77, 16), (1, 1, 260, 112), (1, 16, 384, 40), (1, 1, 1, 72)])
def test_attention_other_head_sizes(hexmi, oracle, case, dtype, causal):
    # head sizes below 128 in multiples of 8 run the matrix-core kernel for 64 or 128 on tiles padded with zero
    # columns; the output buffer starts as NaN and has one row more than the result, which must stay as it is
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, dtype, seed=D + S)
    scale = 1.0 / math.sqrt(D)
    buf = torch.full((Z * H * S + 1, D), float("nan"), dtype=dtype, device="cuda")
    out = buf[:Z * H * S].view(Z, H, S, D)
    hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out=out)
    want = _oracle(oracle, q, k, v, scale, causal)
    tol = 2e-2 if dtype == torch.float16 else 4e-2
    assert (out.cpu().float() - want).abs().max() <= tol
    assert torch.isnan(buf[-1]).all()
    got32 = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    assert (got32 - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [(1, 2, 300, 256), (2, 1, 129, 192), (1, 3, 64, 136), (1, 8, 200, 160), (1, 1, 1000, 200),
                                  (1, 1, 1, 256), (2, 8, 515, 144)])
def test_attention_head_sizes_up_to_256(hexmi, oracle, case, dtype, causal):
    # head sizes above 128 run the kernel for 128 on two halves of the head: the scores sum over both halves' K
    # tiles, the second half is padded like a narrow head
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, dtype, seed=D + S)
    scale = 1.0 / math.sqrt(D)
    buf = torch.full((Z * H * S + 1, D), float("nan"), dtype=dtype, device="cuda")
    out = buf[:Z * H * S].view(Z, H, S, D)
    hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out=out)
    want = _oracle(oracle, q, k, v, scale, causal)
    tol = 2e-2 if dtype == torch.float16 else 4e-2
    assert (out.cpu().float() - want).abs().max() <= tol
    assert torch.isnan(buf[-1]).all()
    got32 = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    assert (got32 - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


def test_attention_padded_head_equals_the_zero_padded_problem(hexmi):
    # head size 80 on the kernel for 128 is the 128-wide problem with 48 zero columns in Q, K and V (and 1/sqrt(80)):
    # the same kernel, the same arithmetic -- bit for bit
    Z, H, S, D = 2, 8, 700, 80
    q, k, v = _qkv(Z, H, S, D, torch.float16, seed=31)
    scale = 1.0 / math.sqrt(D)
    for causal in (False, True):
        got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal).cpu()
        qp, kp, vp = (torch.nn.functional.pad(t, (0, 48)) for t in (q, k, v))
        want = hexmi.flash_attention(qp.cuda(), kp.cuda(), vp.cuda(), scale, causal).cpu()
        assert torch.equal(got, want[..., :D])
        assert (want[..., D:] == 0).all()
    # and head size 192 is the 256-wide problem with 64 zero columns (both on the two-halves form)
    q, k, v = _qkv(1, 8, 400, 192, torch.float16, seed=32)
    scale = 1.0 / math.sqrt(192)
    for causal in (False, True):
        got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal).cpu()
        qp, kp, vp = (torch.nn.functional.pad(t, (0, 64)) for t in (q, k, v))
        want = hexmi.flash_attention(qp.cuda(), kp.cuda(), vp.cuda(), scale, causal).cpu()
        assert torch.equal(got, want[..., :192])
        assert (want[..., 192:] == 0).all()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(1, 1, 1024, 64), (1, 2, 100, 128), (2, 2, 65, 32), (1, 1, 130, 80),
                                  # head sizes 64 and 128 run on the fp32 matrix cores: ragged query and key blocks,
                                  # several workgroups per head, a single row
                                  (2, 3, 333, 64), (1, 2, 515, 128), (1, 1, 1, 64), (3, 1, 129, 128),
                                  # narrower heads in multiples of 4: the same kernels on padded tiles
                                  (1, 2, 300, 4), (2, 1, 257, 36), (1, 3, 200, 100), (1, 1, 640, 124), (2, 2, 129, 72)])
def test_attention_parity_fp32(hexmi, oracle, case, causal):
    # (1,1,1024,64) rand inputs, scale 0.5, non-causal is test_flash_attention.py:20-34,171-213
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, torch.float32, rand=True)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), 0.5, causal).cpu()
    want = _oracle(oracle, q, k, v, 0.5, causal)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 8, 2048, 64), (1, 4, 1536 + 40, 128)])
def test_attention_fp32_larger_and_randn(hexmi, case, causal):
    # N(0,1) operands (scores of both signs, running maxima that move) at sizes with many key blocks. Oracle: the
    # PyTorch CPU call the reference's test uses (test/python/triton/test_flash_attention.py:212), in float64.
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, torch.float32, seed=11)
    scale = 1.0 / math.sqrt(D)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal).cpu()
    want = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=causal,
                                                            scale=scale)
    assert got.dtype == torch.float32
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=2e-6)


def test_reference_call_site(hexmi, oracle):
    Z, H, N_CTX, D_HEAD = 1, 1, 1024, 64
    q, k, v = _qkv(Z, H, N_CTX, D_HEAD, torch.float32, rand=True, seed=1)
    out = torch.zeros_like(q)
    hexmi.kernels.attention_fwd_kernel[(4,)](
        pid1=0, Q=q, K=k, V=v, sm_scale=0.5, Out=out, H=H, N_CTX=N_CTX, BLOCK_M=N_CTX // 4, BLOCK_DMODEL=D_HEAD,
        BLOCK_N=64, STAGE=1, stride_0=H * N_CTX * D_HEAD, stride_1=N_CTX * D_HEAD, stride_2=D_HEAD, stride_3=1,
        enableVectorization=True, enableSplitReduceGeneric=True, enableHVXInlining=True, enableSCFLoopUnroll=True,
        enableMultiThreading=True, enableHexKL=False, enableVTCMTiling=False, enableConvertToHexagonmem=False,
        enableHexagonmemCopyToDMA=False)
    assert torch.allclose(out, _oracle(oracle, q, k, v, 0.5, False), rtol=1e-5, atol=1e-6)


def test_reference_call_site_one_head_per_launch(hexmi, oracle):
    # pid1 = off_hz picks the (z, h) pair a launch computes (test_flash_attention.py:102-105): a loop over Z * H
    # fills the output head by head, and a single launch leaves the other heads untouched
    Z, H, N_CTX, D_HEAD = 2, 3, 256, 64
    q, k, v = _qkv(Z, H, N_CTX, D_HEAD, torch.float32, rand=True, seed=4)
    want = _oracle(oracle, q, k, v, 0.5, False)
    out = torch.full_like(q, -7.0)
    kw = dict(Q=q, K=k, V=v, sm_scale=0.5, Out=out, H=H, N_CTX=N_CTX, BLOCK_M=64, BLOCK_DMODEL=D_HEAD, BLOCK_N=64,
              STAGE=1, stride_0=H * N_CTX * D_HEAD, stride_1=N_CTX * D_HEAD, stride_2=D_HEAD, stride_3=1)
    hexmi.kernels.attention_fwd_kernel[(4,)](pid1=4, **kw)              # z = 1, h = 1
    assert torch.allclose(out[1, 1], want[1, 1], rtol=1e-5, atol=1e-6)
    untouched = torch.ones(Z, H, dtype=torch.bool)
    untouched[1, 1] = False
    assert (out[untouched] == -7.0).all()
    for pid1 in range(Z * H):
        hexmi.kernels.attention_fwd_kernel[(4,)](pid1=pid1, **kw)
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        hexmi.kernels.attention_fwd_kernel[(4,)](pid1=Z * H, **kw)
    all_heads = torch.zeros_like(q)
    hexmi.kernels.attention_fwd_kernel[(4,)](pid1=None, **{**kw, "Out": all_heads})
    assert torch.equal(all_heads, out)


def test_hexkl_attention_fixture_types(hexmi, oracle):
    # test/python/mlir/hexkl_attention: fp16 Q/K/V ~ N(0, 0.5) rounded to 4 decimals, fp32 output, MAX_DIFF 1e-3
    g = _gen(2)
    q, k, v = ((torch.randn(1, 1, 1024, 64, generator=g) * 0.5 * 10000).round() / 10000 for _ in range(3))
    q, k, v = q.half(), k.half(), v.half()
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), 0.5, False, out_dtype=torch.float32).cpu()
    assert (got - _oracle(oracle, q, k, v, 0.5, False)).abs().max() <= 1e-3


def test_causal_invariants(hexmi):
    q, k, v = _qkv(2, 2, 512, 128, torch.float16, seed=3)
    o = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), None, True).cpu()
    assert torch.equal(o[:, :, 0], v[:, :, 0])                            # row 0 attends to key 0 only
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 300:] = 9.0
    v2[:, :, 300:] = -7.0
    o2 = hexmi.flash_attention(q.cuda(), k2.cuda(), v2.cuda(), None, True).cpu()
    assert torch.equal(o2[:, :, :300], o[:, :, :300])                      # later keys never reach earlier rows
    # constant V: any softmax weights give back the constant
    vc = torch.full_like(v, 0.75)
    oc = hexmi.flash_attention(q.cuda(), k.cuda(), vc.cuda(), None, False).cpu()
    assert (oc.float() - 0.75).abs().max() <= 1e-3


@pytest.mark.parametrize("shape", [(4, 32, 4096, 128), (1, 32, 16384, 128)])
def test_attention_config_sizes(hexmi, oracle, shape):
    """Measured configurations (causal fp16). The oracle runs on 3 heads x 48 query rows spread over the
    sequence (all keys each); the whole output is covered by properties: heads are independent (running one
    head alone gives the same bits) and row 0 of every head equals V[0]."""
    from hexmi.workloads import attention_inputs
    Z, H, S, D = shape
    inp = attention_inputs(Z, H, S, D)
    q, k, v, scale = inp["q"], inp["k"], inp["v"], inp["sm_scale"]
    o = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, True).cpu()
    assert torch.equal(o[:, :, 0], v[:, :, 0])
    rows = torch.cat([torch.arange(0, 16), torch.arange(S // 2 - 8, S // 2 + 8), torch.arange(S - 16, S)])
    for (z, h) in [(0, 0), (Z - 1, H - 1), (0, 17)]:
        qh, kh, vh = q[z, h], k[z, h], v[z, h]
        s = (qh[rows].double() @ kh.double().t()) * scale
        mask = torch.arange(S)[None, :] > rows[:, None]
        s = s.masked_fill(mask, float("-inf"))
        want = torch.softmax(s, -1) @ vh.double()
        assert (o[z, h, rows].double() - want).abs().max() <= 2e-2
        one = hexmi.flash_attention(qh[None, None].cuda(), kh[None, None].cuda(), vh[None, None].cuda(), scale, True).cpu()
        assert torch.equal(one[0, 0], o[z, h])
    # cross-check the in-test closed form against the oracle on a short prefix (causal rows see only keys <= row)
    z, h = 0, 0
    P = 192
    want_o = _oracle(oracle, q[z, h, :P][None, None], k[z, h, :P][None, None], v[z, h, :P][None, None], scale, True)
    assert (o[z, h, :P].float() - want_o[0, 0]).abs().max() <= 2e-2


def test_attention_errors(hexmi):
    q = torch.zeros(1, 1, 8, 16, dtype=torch.float16)
    with pytest.raises(ValueError):
        hexmi.flash_attention(q, q[:, :, :4], q)
    with pytest.raises(TypeError):
        hexmi.flash_attention(q, q.float(), q)
    assert hexmi.flash_attention(torch.empty(1, 2, 0, 64, device="cuda", dtype=torch.float16),
                                 torch.empty(1, 2, 0, 64, device="cuda", dtype=torch.float16),
                                 torch.empty(1, 2, 0, 64, device="cuda", dtype=torch.float16)).shape == (1, 2, 0, 64)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("scale", [0.0, -0.3])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_attention_zero_and_negative_scale(hexmi, oracle, dtype, scale, causal):
    # the matrix-core kernels take the row maximum before scaling, which is right for a positive scale only: other
    # scales must still give softmax(scale * Q K^T) V (scale 0: the mean of the visible V rows)
    q, k, v = _qkv(1, 2, 200, 128, dtype, seed=11)
    o = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    want = _oracle(oracle, q, k, v, scale, causal)
    assert torch.isfinite(o).all()
    assert (o - want).abs().max() <= (2e-2 if dtype == torch.float16 else 1e-5 * want.abs().max())
    if scale == 0.0 and not causal:
        assert (o - v.float().mean(2, keepdim=True)).abs().max() <= 2e-3


def test_attention_head_size_256(hexmi, oracle):
    q, k, v = _qkv(1, 2, 70, 256, torch.float16, seed=12)
    o = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), 1 / 16.0, True, out_dtype=torch.float32).cpu()
    assert (o - _oracle(oracle, q, k, v, 1 / 16.0, True)).abs().max() <= 2e-2


# ---- tm_tensor.attention: [B, S, D] operands, rectangular scores, additive mask -----------------------------
def _oracle_masked(oracle, q, k, v, mask, scale):
    qn, tag = to_np(q)
    kn, _ = to_np(k)
    vn, _ = to_np(v)
    mn = None if mask is None else to_np(mask)[0]
    return torch.from_numpy(oracle.attention_masked(qn, kn, vn, mn, scale, out_dtype=np.float32, dtype=tag))


def _mask(B, Sq, Skv, dtype, seed, drop=0.3):
    g = _gen(seed)
    m = torch.randn(B, Sq, Skv, generator=g)
    m[torch.rand(B, Sq, Skv, generator=g) < drop] = float("-inf")
    m[:, :, 0] = 0.0                                   # every row keeps a key
    return m.to(dtype)


MASKED_CASES = [(2, 128, 128, 128), (3, 200, 72, 64), (1, 1, 64, 128), (2, 77, 516, 128), (1, 300, 4, 64),
                (1, 130, 1024, 128), (2, 65, 66, 64), (1, 40, 100, 80),   # the last two: Skv % 4 != 0 / other D
                # more than 128 queries and Skv % 8 == 0: mask tiles staged through LDS by 256-row workgroups
                # (ragged last row block, ragged last key block, several row blocks, many batch entries)
                (3, 300, 520, 128), (2, 513, 72, 64), (1, 257, 2048 + 8, 128), (40, 129, 136, 64),
                # head sizes below 128 in multiples of 8: the 128-row kernel on tiles padded with zero columns
                (2, 200, 72, 80), (1, 300, 520, 96), (3, 129, 136, 32), (1, 77, 516, 40), (2, 64, 64, 112),
                # key counts that are not multiples of 4 (matrix-core kernel without a mask, row-wise with one)
                (4, 1024, 77, 64), (2, 300, 1, 128), (1, 129, 515, 80)]


@pytest.mark.parametrize("with_mask", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", MASKED_CASES)
def test_masked_attention_parity_half(hexmi, oracle, case, dtype, with_mask):
    B, Sq, Skv, D = case
    g = _gen(21)
    q = torch.randn(B, Sq, D, generator=g).to(dtype)
    k, v = torch.randn(B, Skv, D, generator=g).to(dtype), torch.randn(B, Skv, D, generator=g).to(dtype)
    mask = _mask(B, Sq, Skv, dtype, 22) if with_mask else None
    scale = 1.0 / math.sqrt(D)
    got = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda()).cpu()
    want = _oracle_masked(oracle, q, k, v, mask, scale)
    assert got.dtype == dtype and got.shape == (B, Sq, D)
    assert (got.float() - want).abs().max() <= (2e-2 if dtype == torch.float16 else 4e-2)
    got32 = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), None if mask is None else mask.cuda(),
                            out_dtype=torch.float32).cpu()
    assert (got32 - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


@pytest.mark.parametrize("case", [(2, 50, 70, 32), (1, 64, 64, 128), (1, 33, 129, 64),
                                  # Skv % 4 == 0 with head size 64 / 128: the fp32 matrix-core kernel with a mask
                                  (2, 200, 72, 64), (1, 130, 516, 128), (3, 129, 1028, 64),
                                  # ... and narrower heads on padded tiles
                                  (2, 200, 72, 80), (1, 130, 516, 36), (2, 129, 132, 100)])
def test_masked_attention_parity_fp32(hexmi, oracle, case):
    B, Sq, Skv, D = case
    g = _gen(23)
    q, k, v = torch.rand(B, Sq, D, generator=g), torch.rand(B, Skv, D, generator=g), torch.rand(B, Skv, D, generator=g)
    mask = _mask(B, Sq, Skv, torch.float32, 24)
    got = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), mask.cuda()).cpu()
    want = _oracle_masked(oracle, q, k, v, mask, 1.0 / math.sqrt(D))
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_masked_attention_properties(hexmi):
    # a causal additive mask reproduces the causal kernel; a constant added to the mask changes nothing;
    # host tensors are staged and `out` is filled in place
    B, S, D = 2, 256, 128
    g = _gen(25)
    q, k, v = (torch.randn(B, S, D, generator=g).half() for _ in range(3))
    tri = torch.full((S, S), float("-inf")).triu(1).half().expand(B, S, S).contiguous()
    got = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), tri.cuda()).cpu()
    causal = hexmi.flash_attention(q.view(B, 1, S, D).cuda(), k.view(B, 1, S, D).cuda(), v.view(B, 1, S, D).cuda(),
                                   None, True).cpu().view(B, S, D)
    assert (got.float() - causal.float()).abs().max() <= 2e-3
    shifted = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), (tri + 2.0).cuda()).cpu()
    assert (shifted.float() - got.float()).abs().max() <= 2e-3
    out = torch.empty(B, S, D, dtype=torch.float16)
    ret = hexmi.attention(q, k, v, tri, out=out)
    assert ret is out and torch.equal(out, got)
    with pytest.raises(ValueError):
        hexmi.attention(q, k, v, tri[:, :, :-4])


def test_masked_attention_fully_masked_row_is_nan(hexmi):
    # LowerTmTensor.cpp:164-222: max = -inf, x - max = nan, exp / sum / div propagate it
    B, S, D = 1, 64, 64
    g = _gen(26)
    q, k, v = (torch.randn(B, S, D, generator=g).half() for _ in range(3))
    mask = torch.zeros(B, S, S).half()
    mask[0, 5, :] = float("-inf")
    got = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), mask.cuda()).cpu()
    assert torch.isnan(got[0, 5]).all() and not torch.isnan(got[0, :5]).any() and not torch.isnan(got[0, 6:]).any()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", [(2, 200, 320, 128, 40), (1, 130, 260, 64, 70)])
def test_masked_attention_window_mask(hexmi, oracle, case, dtype):
    # a band mask (-inf outside a window that ends past the row index): most rows have every key of their first
    # 64-key blocks masked out, so the running maximum is still -inf when the first finite score arrives
    B, Sq, Skv, D, width = case
    g = _gen(31)
    q = torch.randn(B, Sq, D, generator=g).to(dtype)
    k, v = torch.randn(B, Skv, D, generator=g).to(dtype), torch.randn(B, Skv, D, generator=g).to(dtype)
    rows, cols = torch.arange(Sq)[:, None], torch.arange(Skv)[None, :]
    keep = (cols > rows + 60 - width) & (cols <= rows + 60)
    mask = torch.zeros(Sq, Skv).masked_fill(~keep, float("-inf")).to(dtype).expand(B, Sq, Skv).contiguous()
    scale = 1.0 / math.sqrt(D)
    got = hexmi.attention(q.cuda(), k.cuda(), v.cuda(), mask.cuda()).cpu()
    want = _oracle_masked(oracle, q, k, v, mask, scale)
    assert not torch.isnan(got).any()
    assert (got.float() - want).abs().max() <= (2e-2 if dtype == torch.float16 else 4e-2)


@pytest.mark.parametrize("case", [(1, 1, 8200, 64, True), (1, 1, 8192, 128, False), (1, 2, 8192 + 130, 128, True)])
def test_attention_long_sequences(hexmi, oracle, case):
    # long sequences, few heads (too few 256-row workgroups to fill the chip: 128-row workgroups)
    Z, H, S, D, causal = case
    q, k, v = _qkv(Z, H, S, D, torch.float16, seed=7)
    scale = 1.0 / math.sqrt(D)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal).cpu()
    want = _oracle(oracle, q, k, v, scale, causal)
    assert (got.float() - want).abs().max() <= 2e-2
    # rows of different 256-row blocks do not interact: the first 300 rows of a causal run equal a 300-row run
    if causal:
        short = hexmi.flash_attention(q[:, :, :300].contiguous().cuda(), k[:, :, :300].contiguous().cuda(),
                                      v[:, :, :300].contiguous().cuda(), scale, True).cpu()
        assert (short.float() - got[:, :, :300].float()).abs().max() <= 2e-3


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 16, 2048 + 70, 128, torch.float16), (1, 40, 2048, 64, torch.float16),
                                  (4, 8, 2304, 128, torch.bfloat16), (1, 8, 8192 + 130, 128, torch.float16)])
def test_attention_256_row_workgroups(hexmi, case, causal):
    # from 2048 keys on, grids with at least one 256-row block per CU run 8-wave workgroups (256 query rows per
    # K/V tile copy): ragged lengths, head counts off the XCD multiple, both dtypes. Oracle: the PyTorch CPU call
    # the reference's test uses (test/python/triton/test_flash_attention.py:212).
    Z, H, S, D, dtype = case
    q, k, v = _qkv(Z, H, S, D, dtype, seed=9)
    scale = 1.0 / math.sqrt(D)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal,
                                                            scale=scale)
    assert (got - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 52, 2048, torch.float16), (1, 100, 2048 + 40, torch.bfloat16)])
def test_attention_three_workgroups_per_cu(hexmi, case, causal):
    # D = 64 between 2048 and 4095 keys with six or more 128-row units per CU runs three 128-row workgroups per CU
    # (a persistent grid of 768): head counts off the XCD multiple, a ragged length, both dtypes. Oracle: the
    # PyTorch CPU call the reference's test uses (test/python/triton/test_flash_attention.py:212).
    Z, H, S, dtype = case
    q, k, v = _qkv(Z, H, S, 64, dtype, seed=13)
    scale = 1.0 / math.sqrt(64)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal,
                                                            scale=scale)
    assert (got - want).abs().max() <= (5e-3 if dtype == torch.float16 else 3e-2)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("case", [(2, 36, 1280, 64), (1, 72, 1024, 128), (5, 13, 777, 128)])
def test_attention_more_units_than_resident_workgroups(hexmi, case, causal):
    # more (head, query block) units than the persistent grid holds, head counts that are and are not multiples of
    # the 8 XCDs, ragged lengths: every unit must be visited exactly once. Oracle: the PyTorch CPU call the
    # reference's test uses (test/python/triton/test_flash_attention.py:212).
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, torch.float16, seed=5)
    scale = 1.0 / math.sqrt(D)
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, causal, out_dtype=torch.float32).cpu()
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal,
                                                            scale=scale)
    assert (got - want).abs().max() <= 5e-3


@pytest.mark.parametrize("case", [(1, 32, 3840, 128), (1, 32, 2176, 128), (1, 24, 5120, 128), (1, 64, 2176, 64)])
def test_causal_attention_block_counts_off_the_power_of_two(hexmi, case):
    # causal units of unequal length are dealt to the persistent workgroups in groups of heads, longest first and
    # padded to whole passes (15, 9, 20 query blocks of 256 rows on 32 workgroups per XCD; 17 blocks of 128 rows on
    # 96): every unit must be visited exactly once, so the output starts as NaN. Oracle: the PyTorch CPU call the
    # reference's test uses (test/python/triton/test_flash_attention.py:212).
    Z, H, S, D = case
    q, k, v = _qkv(Z, H, S, D, torch.float16, seed=21)
    scale = 1.0 / math.sqrt(D)
    out = torch.full((Z, H, S, D), float("nan"), dtype=torch.float32, device="cuda")
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), scale, True, out=out).cpu()
    assert not torch.isnan(got).any()
    want = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True, scale=scale)
    assert (got - want).abs().max() <= 5e-3
