"""GPU parity of softmax / RMSNorm / LayerNorm against the CPU oracle, through the C ABI (hexmi.ops -> ctypes).

Tolerances: fp32 results within rel-err 1e-5 of the oracle; fp16 / bf16 results within one unit in the last
place of the oracle's rounded value (both round the same real number; the kernel's fp32 arithmetic may land on
the other side of a rounding boundary), with an absolute floor where the value is a cancellation residue.
"""
import numpy as np
import pytest
import torch

from util import close16, from_np, to_np

pytestmark = pytest.mark.gpu

F32_RTOL = 1e-5


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _check(got, want, dtype, atol16=1e-6, atol32=1e-7):
    got = got.cpu()
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=F32_RTOL, atol=atol32), (got - want).abs().max()
    else:
        assert close16(got, want, max_ulp=1, atol=atol16)


SOFTMAX_SHAPES = [(128, 128), (4, 65536), (37, 513), (3, 5), (1, 1), (64, 1024), (5, 4096), (2, 20000), (7, 100001)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
def test_softmax_parity(hexmi, oracle, dtype, shape):
    x = (torch.randn(*shape, generator=_gen(0)) * 3).to(dtype)
    a, tag = to_np(x)
    want = from_np(oracle.softmax(a, dtype=tag), dtype)
    got = hexmi.softmax(x.cuda())
    _check(got, want, dtype, atol16=1e-7)


def test_softmax_config_shape_and_properties(hexmi, oracle):
    # the measured configuration: fp32 [4096, 1024], N(0,1), seed 0
    from hexmi.workloads import softmax_inputs
    x = softmax_inputs()["x"]
    got = hexmi.softmax(x.cuda()).cpu()
    want = torch.from_numpy(oracle.softmax(x.numpy()))
    assert torch.allclose(got, want, rtol=F32_RTOL, atol=1e-9)
    assert torch.allclose(got.sum(-1), torch.ones(4096), atol=1e-5)
    got_shift = hexmi.softmax((x + 2.5).cuda()).cpu()
    assert torch.allclose(got_shift, got, rtol=1e-5, atol=1e-8)


def test_softmax_strided_rows_and_out(hexmi, oracle):
    x = torch.randn(33, 256, generator=_gen(1))
    big = torch.zeros(33, 512, device="cuda")
    big[:, :256] = x.cuda()
    view = big[:, :256]                       # leading dimension 512
    out = torch.full((33, 512), -1.0, device="cuda")
    torch.ops.hexmi.softmax(view, out[:, :256])
    want = torch.from_numpy(oracle.softmax(x.numpy()))
    assert torch.allclose(out[:, :256].cpu(), want, rtol=F32_RTOL, atol=1e-9)
    assert (out[:, 256:] == -1.0).all()       # nothing written past the row


def test_softmax_host_tensors_in_place(hexmi, oracle):
    # reference call convention: host tensors, preallocated output written in place
    x = torch.rand(128, 128, generator=_gen(2))
    out = torch.empty_like(x)
    hexmi.kernels.softmax_kernel[(4,)](x, out, NUM_ROWS=128, NUM_COLS=128, BLOCK_SIZE=128,
                                       enableMultiThreading=False, enableVTCMTiling=False,
                                       enableConvertToHexagonmem=False, enableHexagonmemCopyToDMA=False,
                                       enableHVXInlining=True, enableSCFLoopUnroll=True,
                                       enableSplitReduceGeneric=True)
    assert torch.allclose(out, torch.from_numpy(oracle.softmax(x.numpy())), atol=1e-5)   # test_softmax.py ATOL_FP32
    out2 = torch.empty_like(x)
    hexmi.kernels.online_softmax[(4,)](x, out2, NUM_ROWS=128, NUM_COLS=128, BLOCK_SIZE=32)
    assert torch.equal(out, out2)


def test_softmax_extreme_values(hexmi):
    x = torch.tensor([[1e4, 1e4 - 1, -1e4, 0.0], [-float("inf"), 0.0, 0.0, -float("inf")]], device="cuda")
    y = hexmi.softmax(x).cpu()
    e = float(np.exp(-1.0))
    assert torch.allclose(y[0], torch.tensor([1 / (1 + e), e / (1 + e), 0.0, 0.0], dtype=torch.float32), atol=1e-6)
    assert torch.allclose(y[1], torch.tensor([0.0, 0.5, 0.5, 0.0]))


NORM_SHAPES = [(127, 513), (27, 8192), (128, 128), (33, 4096), (5, 24), (3, 7), (2, 16384), (2, 70000), (1, 8)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", NORM_SHAPES)
def test_rms_norm_parity(hexmi, oracle, dtype, shape):
    g = _gen(3)
    x = torch.randn(*shape, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(shape[1], generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, _ = to_np(w)
    want = from_np(oracle.rms_norm(a, wn, 1e-5, dtype=tag), dtype)
    got = hexmi.rms_norm(x.cuda(), w.cuda(), 1e-5)
    _check(got, want, dtype)
    got_now = hexmi.rms_norm(x.cuda(), None, 1e-5)
    want_now = from_np(oracle.rms_norm(a, None, 1e-5, dtype=tag), dtype)
    _check(got_now, want_now, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", NORM_SHAPES)
def test_layer_norm_parity(hexmi, oracle, dtype, shape):
    g = _gen(4)
    x = (torch.randn(*shape, generator=g) + 0.5).to(dtype)
    w = (1 + 0.1 * torch.randn(shape[1], generator=g)).to(dtype)
    b = (0.1 * torch.randn(shape[1], generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, _ = to_np(w)
    bn, _ = to_np(b)
    want, mean, rstd = oracle.layer_norm(a, wn, bn, 1e-5, dtype=tag)
    want = from_np(want, dtype)
    m = torch.empty(shape[0], device="cuda")
    r = torch.empty(shape[0], device="cuda")
    got = hexmi.layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-5, mean=m, rstd=r)
    _check(got, want, dtype, atol16=2e-6, atol32=2e-6)      # x_hat*w + b near zero carries the rounding of its terms
    assert torch.allclose(m.cpu(), torch.from_numpy(mean), rtol=1e-5, atol=1e-6)
    assert torch.allclose(r.cpu(), torch.from_numpy(rstd), rtol=1e-5)


def test_norm_config_shape(hexmi, oracle):
    # the measured configuration: fp16 [8192, 4096], w ~ N(1, 0.1), b ~ N(0, 0.1), eps 1e-5
    from hexmi.workloads import norm_inputs
    inp = norm_inputs()
    x, w, b = inp["x"], inp["weight"], inp["bias"]
    got_r = hexmi.rms_norm(x.cuda(), w.cuda(), 1e-5).cpu()
    got_l = hexmi.layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-5).cpu()
    want_r = torch.from_numpy(oracle.rms_norm(x.numpy(), w.numpy(), 1e-5))
    want_l = torch.from_numpy(oracle.layer_norm(x.numpy(), w.numpy(), b.numpy(), 1e-5)[0])
    assert close16(got_r, want_r, 1, 1e-6)
    assert close16(got_l, want_l, 1, 2e-6)
    # size-independent properties: scale equivariance of RMSNorm direction, shift invariance of LayerNorm
    got_r2 = hexmi.rms_norm((x * 2).cuda(), w.cuda(), 4e-5).cpu()
    assert close16(got_r2, got_r, 1, 1e-6)


# Shapes that fill a tile exactly and are tall enough for the persistent walk (a few workgroups per CU, each
# walking several row groups with the next group's loads in flight); row counts chosen so that workgroups walk
# unequal numbers of groups.
WALK_SHAPES = [(torch.float16, 32772, 512), (torch.float16, 16388, 1024), (torch.float32, 8204, 1024),
               (torch.float32, 16400, 1024),       # softmax over >= 16384 rows: one workgroup per CU in the walk
               (torch.float16, 4100, 4096), (torch.bfloat16, 2051, 8192), (torch.float32, 1030, 8192)]


@pytest.mark.parametrize("dtype,rows,cols", WALK_SHAPES)
def test_persistent_walk(hexmi, oracle, dtype, rows, cols):
    g = _gen(11)
    x = (torch.randn(rows, cols, generator=g) + 0.25).to(dtype)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    b = (0.1 * torch.randn(cols, generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, _ = to_np(w)
    bn, _ = to_np(b)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    _check(hexmi.softmax(xd), from_np(oracle.softmax(a, dtype=tag), dtype), dtype, atol16=1e-7)
    _check(hexmi.rms_norm(xd, wd, 1e-5), from_np(oracle.rms_norm(a, wn, 1e-5, dtype=tag), dtype), dtype)
    _check(hexmi.rms_norm(xd, None, 1e-5), from_np(oracle.rms_norm(a, None, 1e-5, dtype=tag), dtype), dtype)
    want, mean, rstd = oracle.layer_norm(a, wn, bn, 1e-5, dtype=tag)
    m = torch.full((rows,), float("nan"), device="cuda")
    r = torch.full((rows,), float("nan"), device="cuda")
    got = hexmi.layer_norm(xd, wd, bd, 1e-5, mean=m, rstd=r)
    _check(got, from_np(want, dtype), dtype, atol16=2e-6, atol32=2e-6)
    assert torch.allclose(m.cpu(), torch.from_numpy(mean), rtol=1e-5, atol=1e-6)
    assert torch.allclose(r.cpu(), torch.from_numpy(rstd), rtol=1e-5)
    want_plain = oracle.layer_norm(a, None, None, 1e-5, dtype=tag)[0]
    _check(hexmi.layer_norm(xd, None, None, 1e-5), from_np(want_plain, dtype), dtype, atol16=2e-6, atol32=2e-6)


def test_norm_reference_call_sites(hexmi, oracle):
    g = _gen(5)
    # test_rms_norm.py:65-89
    x = torch.rand(127, 513, generator=g)
    wt = torch.rand(513, generator=g)
    out = torch.empty_like(x)
    hexmi.kernels.rms_norm_fwd_kernel[(4,)](x, out, wt, EPSILON=1e-5, NUM_ROWS=127, NUM_COLS=513, BLOCK_SIZE=1024,
                                            enableMultiThreading=False, enableVTCMTiling=False,
                                            enableConvertToHexagonmem=False, enableHexagonmemCopyToDMA=True)
    assert torch.allclose(out, torch.from_numpy(oracle.rms_norm(x.numpy(), wt.numpy(), 1e-5)), atol=1e-2)
    assert torch.allclose(out, torch.from_numpy(oracle.rms_norm(x.numpy(), wt.numpy(), 1e-5)), rtol=1e-5, atol=1e-7)
    # test_layer_norm.py:84-115
    x = torch.rand(27, 8192, generator=g)
    wt = torch.rand(8192, generator=g)
    bs = torch.rand(8192, generator=g)
    out = torch.empty_like(x)
    means = torch.empty(27)
    rstds = torch.empty(27)
    hexmi.kernels.layer_norm_fwd_kernel[(4,)](x, out, wt, bs, means, rstds, EPSILON=1e-5, NUM_ROWS=27, NUM_COLS=8192,
                                              BLOCK_SIZE=8192, enableMultiThreading=False)
    want, mean, rstd = oracle.layer_norm(x.numpy(), wt.numpy(), bs.numpy(), 1e-5)
    assert torch.allclose(out, torch.from_numpy(want), atol=1e-5)
    assert torch.allclose(means, torch.from_numpy(mean), atol=1e-6)
    assert torch.allclose(rstds, torch.from_numpy(rstd), rtol=1e-5)


def test_empty_inputs(hexmi):
    assert hexmi.softmax(torch.empty(0, 16, device="cuda")).shape == (0, 16)
    assert hexmi.rms_norm(torch.empty(0, 16, device="cuda", dtype=torch.float16)).shape == (0, 16)
    assert hexmi.layer_norm(torch.empty(4, 0, device="cuda")).shape == (4, 0)
