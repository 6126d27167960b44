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
    # test_online_softmax.py:84-113: four programs, BLOCK_ROW_SIZE = BLOCK_COL_SIZE = 32, ATOL 1e-5
    out2 = torch.empty_like(x)
    hexmi.kernels.online_softmax[(4,)](x, out2, NUM_ROWS=128, NUM_COLS=128, BLOCK_ROW_SIZE=32, BLOCK_COL_SIZE=32,
                                       enableMultiThreading=False, enableVTCMTiling=False,
                                       enableConvertToHexagonmem=False, enableHexagonmemCopyToDMA=False)
    assert torch.allclose(out2, torch.from_numpy(oracle.online_softmax_f32(x.numpy(), 32)), rtol=F32_RTOL, atol=1e-9)
    assert torch.allclose(out2, out, rtol=F32_RTOL, atol=1e-9)


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


# ---- rows split over several workgroups (the online / split-reduction form) ------------------------------------

# shapes the library splits by itself: few long rows (the reference's 4 x 65536 of
# test_softmax_scf_multithread.py:19-24) and rows beyond 128 KiB, whole and ragged last parts
SPLIT_SHAPES = [(torch.float32, 4, 65536), (torch.float16, 4, 65536), (torch.float32, 16, 131072),
                (torch.float32, 1, 1 << 20), (torch.float16, 3, 40000), (torch.float32, 2, 100004),
                (torch.bfloat16, 5, 70000), (torch.float32, 300, 40000)]


@pytest.mark.parametrize("dtype,rows,cols", SPLIT_SHAPES)
def test_split_rows_parity(hexmi, oracle, dtype, rows, cols):
    assert hexmi.lib().hexmi_row_workspace(rows, cols, 0, hexmi.ops._dt(torch.empty(0, dtype=dtype))) > 0
    g = _gen(21)
    x = (torch.randn(rows, cols, generator=g) * 2 + 0.25).to(dtype)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    b = (0.1 * torch.randn(cols, generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, _ = to_np(w)
    bn, _ = to_np(b)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    _check(hexmi.softmax(xd), from_np(oracle.softmax(a, dtype=tag), dtype), dtype, atol16=1e-7, atol32=1e-12)
    _check(hexmi.rms_norm(xd, wd, 1e-5), from_np(oracle.rms_norm(a, wn, 1e-5, dtype=tag), dtype), dtype)
    want, mean, rstd = oracle.layer_norm(a, wn, bn, 1e-5, dtype=tag)
    m = torch.full((rows,), float("nan"), device="cuda")
    r = torch.full((rows,), float("nan"), device="cuda")
    got = hexmi.layer_norm(xd, wd, bd, 1e-5, mean=m, rstd=r)
    _check(got, from_np(want, dtype), dtype, atol16=2e-6, atol32=2e-6)
    assert torch.allclose(m.cpu(), torch.from_numpy(mean), rtol=1e-5, atol=1e-6)
    assert torch.allclose(r.cpu(), torch.from_numpy(rstd), rtol=1e-5)
    # rows sum to one; a shift of the row changes nothing (softmax), nor does it change LayerNorm
    sm = hexmi.softmax(xd).float().sum(-1).cpu()
    assert torch.allclose(sm, torch.ones(rows), atol=2e-3 if dtype != torch.float32 else 1e-5)


@pytest.mark.parametrize("dtype,rows,cols,block", [(torch.float32, 128, 128, 32), (torch.float32, 37, 520, 24),
                                                   (torch.float16, 37, 520, 24), (torch.float32, 5, 4096, 1000),
                                                   (torch.float16, 64, 8192, 2048), (torch.bfloat16, 9, 1024, 1024),
                                                   (torch.float32, 6, 100000, 100000)])
def test_forced_column_blocks(hexmi, oracle, dtype, rows, cols, block):
    g = _gen(22)
    x = (torch.randn(rows, cols, generator=g) * 3).to(dtype)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    b = (0.1 * torch.randn(cols, generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, _ = to_np(w)
    bn, _ = to_np(b)
    xd = x.cuda()
    got = hexmi.softmax(xd, block_cols=block)
    _check(got, from_np(oracle.softmax(a, dtype=tag), dtype), dtype, atol16=1e-7, atol32=1e-12)
    if dtype == torch.float32 and cols % block == 0 and cols <= 8192:
        # the reference's two-phase algorithm restated with the same block size (its fp32 running sums, so short rows)
        assert torch.allclose(got.cpu(), torch.from_numpy(oracle.online_softmax_f32(a, block)), rtol=F32_RTOL, atol=1e-12)
    _check(hexmi.rms_norm(xd, w.cuda(), 1e-5, block_cols=block), from_np(oracle.rms_norm(a, wn, 1e-5, dtype=tag), dtype), dtype)
    want, mean, rstd = oracle.layer_norm(a, wn, bn, 1e-5, dtype=tag)
    m = torch.empty(rows, device="cuda")
    r = torch.empty(rows, device="cuda")
    got = hexmi.layer_norm(xd, w.cuda(), b.cuda(), 1e-5, mean=m, rstd=r, block_cols=block)
    _check(got, from_np(want, dtype), dtype, atol16=2e-6, atol32=2e-6)
    assert torch.allclose(m.cpu(), torch.from_numpy(mean), rtol=1e-5, atol=1e-6)
    assert torch.allclose(r.cpu(), torch.from_numpy(rstd), rtol=1e-5)


def test_split_softmax_rows_of_minus_infinity(hexmi):
    # whole column blocks of -inf (masked scores): they add nothing; a row of nothing else is NaN, as torch gives
    x = torch.randn(3, 65536, generator=_gen(23))
    x[0, :40000] = -float("inf")
    x[1, 1024:] = -float("inf")
    x[2, :] = -float("inf")
    got = hexmi.softmax(x.cuda()).cpu()
    want = torch.softmax(x.double(), -1).float()
    assert torch.allclose(got[:2], want[:2], rtol=F32_RTOL, atol=1e-12)
    assert torch.isnan(got[2]).all() and torch.isnan(want[2]).all()


@pytest.mark.parametrize("split", [False, True])
def test_norms_on_strided_rows(hexmi, oracle, split):
    # rows inside wider buffers (leading dimension > cols), read and written in place
    rows, cols, ld = (4, 65536, 65536 + 64) if split else (33, 512, 768)
    g = _gen(24)
    x = torch.randn(rows, cols, generator=g).half()
    w = (1 + 0.1 * torch.randn(cols, generator=g)).half()
    b = (0.1 * torch.randn(cols, generator=g)).half()
    big = torch.zeros(rows, ld, dtype=torch.float16, device="cuda")
    big[:, :cols] = x.cuda()
    out = torch.full((rows, ld), -1.0, dtype=torch.float16, device="cuda")
    hexmi.rms_norm(big[:, :cols], w.cuda(), 1e-5, out=out[:, :cols])
    assert close16(out[:, :cols].cpu(), torch.from_numpy(oracle.rms_norm(x.numpy(), w.numpy(), 1e-5)), 1, 1e-6)
    assert (out[:, cols:] == -1.0).all()
    out.fill_(-1.0)
    m = torch.empty(rows, device="cuda")
    r = torch.empty(rows, device="cuda")
    hexmi.layer_norm(big[:, :cols], w.cuda(), b.cuda(), 1e-5, out=out[:, :cols], mean=m, rstd=r)
    want, mean, rstd = oracle.layer_norm(x.numpy(), w.numpy(), b.numpy(), 1e-5)
    assert close16(out[:, :cols].cpu(), torch.from_numpy(want), 1, 2e-6)
    assert (out[:, cols:] == -1.0).all()
    assert torch.allclose(m.cpu(), torch.from_numpy(mean), rtol=1e-5, atol=1e-6)
    out.fill_(-1.0)
    hexmi.softmax(big[:, :cols], out=out[:, :cols])
    assert close16(out[:, :cols].cpu(), torch.from_numpy(oracle.softmax(x.numpy())), 1, 1e-7)
    assert (out[:, cols:] == -1.0).all()


def test_row_workspace_contract(hexmi):
    lib = hexmi.lib()
    F32 = hexmi._lib.F32
    assert lib.hexmi_row_workspace(4096, 1024, 0, F32) == 0           # single pass
    assert lib.hexmi_row_workspace(4096, 1024, 256, F32) == 4096 * 4 * 8
    need = lib.hexmi_row_workspace(4, 65536, 0, F32)
    assert need > 0 and need % (4 * 8) == 0
    x = torch.randn(4, 65536, device="cuda")
    y = torch.empty_like(x)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.hexmi_softmax_ws(x.data_ptr(), y.data_ptr(), 4, 65536, 65536, 65536, 0, F32, ws.data_ptr(), need - 1, st) \
        == hexmi._lib.EINVAL
    assert lib.hexmi_softmax_ws(x.data_ptr(), y.data_ptr(), 4, 65536, 65536, 65536, 0, F32, ws.data_ptr(), need, st) == 0
    y2 = torch.empty_like(x)
    assert lib.hexmi_softmax_ws(x.data_ptr(), y2.data_ptr(), 4, 65536, 65536, 65536, 0, F32, None, 0, st) == 0
    torch.cuda.synchronize()
    assert torch.allclose(y, y2, rtol=F32_RTOL, atol=1e-12)
    assert lib.hexmi_softmax_ws(x.data_ptr(), y.data_ptr(), 4, 65536, 100, 65536, 0, F32, None, 0, st) == hexmi._lib.EINVAL


def test_norm_statistics_at_the_edges_of_the_range(hexmi):
    # a sum of squares that overflows (rstd = 0), a row of zeros with eps = 0 (rstd = inf): what torch gives
    import torch.nn.functional as F
    x = torch.zeros(4, 1024)
    x[0] = 1e20
    x[1] = torch.randn(1024, generator=_gen(25))
    x[3] = 3.0                                                     # constant row: zero variance
    for eps in (1e-5, 0.0):
        got = hexmi.rms_norm(x.cuda(), None, eps).cpu()
        want = F.rms_norm(x, (1024,), None, eps)
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-7, equal_nan=True)
        m = torch.empty(4, device="cuda")
        r = torch.empty(4, device="cuda")
        got = hexmi.layer_norm(x.cuda(), None, None, eps, mean=m, rstd=r).cpu()
        want = F.layer_norm(x, (1024,), None, None, eps)
        assert torch.allclose(got[1:], want[1:], rtol=1e-5, atol=1e-6, equal_nan=True)
        var = x.double().var(-1, unbiased=False)
        assert torch.allclose(r.cpu()[1:].double(), 1.0 / torch.sqrt(var + eps)[1:], rtol=1e-5, equal_nan=True)


RAGGED_COLS = [1, 7, 9, 63, 513, 1001, 2049, 4097, 8200 + 3, 12289, 32001, 50257]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cols", RAGGED_COLS)
def test_rows_that_are_not_whole_chunks(hexmi, oracle, dtype, cols):
    # every tile of the one-pass kernel with per-element masks: rows of any length that start at any alignment of the
    # element type (row r starts r * cols elements in), against the oracle; the output is a window between margins
    rows = 9 if cols < 20000 else 3
    g = _gen(cols)
    x = (torch.randn(rows, cols, generator=g) * 2 + 0.3).to(dtype)
    w = (1 + 0.1 * torch.randn(cols, generator=g)).to(dtype)
    b = (0.1 * torch.randn(cols, generator=g)).to(dtype)
    a, tag = to_np(x)
    wn, bn = to_np(w)[0], to_np(b)[0]

    def window(lead=32):
        buf = torch.full((rows * cols + 64,), 5.0, dtype=dtype, device="cuda")
        return buf, buf[lead:lead + rows * cols].view(rows, cols)

    # softmax: output rows as far off the 16-byte boundaries as the input's (whole aligned chunks over the span that
    # covers a row), then three elements further (accesses at the alignment of the element type)
    want_sm = from_np(oracle.softmax(a, dtype=tag), dtype)
    for lead in (32, 35):
        buf, out = window(lead)
        hexmi.softmax(x.cuda(), out=out)
        _check(out, want_sm, dtype, atol16=1e-7)
        assert (buf[:lead] == 5.0).all() and (buf[lead + rows * cols:] == 5.0).all()
    buf, out = window()
    hexmi.rms_norm(x.cuda(), w.cuda(), 1e-5, out=out)
    _check(out, from_np(oracle.rms_norm(a, wn, 1e-5, dtype=tag), dtype), dtype)
    assert (buf[:32] == 5.0).all() and (buf[32 + rows * cols:] == 5.0).all()
    buf, out = window()
    mean = torch.empty(rows, device="cuda")
    rstd = torch.empty(rows, device="cuda")
    hexmi.layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-5, out=out, mean=mean, rstd=rstd)
    want, want_mean, want_rstd = oracle.layer_norm(a, wn, bn, 1e-5, dtype=tag)
    _check(out, from_np(want, dtype), dtype, atol16=2e-6, atol32=2e-6)
    assert (buf[:32] == 5.0).all() and (buf[32 + rows * cols:] == 5.0).all()
    assert torch.allclose(mean.cpu(), torch.from_numpy(want_mean), rtol=1e-5, atol=1e-6)
    assert torch.allclose(rstd.cpu(), torch.from_numpy(want_rstd), rtol=1e-5)

