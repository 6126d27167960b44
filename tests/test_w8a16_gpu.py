"""GPU parity of the weight-only int8 GEMM. The reference has no such kernel (parity unpinned there); the
oracle is the closed form pinned in tests/test_oracle.py. Integer side (dequantisation, scale selection, weight
indexing) is checked bit-exactly; the fp16 result within one unit in the last place of the oracle (or 2e-4
absolute where it is a cancellation residue of partial sums in the thousands), and within 2e-2 after scaling by
1/sqrt(K): outputs reach |c| ~ 100 where one fp16 unit in the last place is 0.06, so a flat 2e-2 cannot hold for
any fp16 result."""
import math
import numpy as np
import pytest
import torch

from util import close16

pytestmark = pytest.mark.gpu


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _inputs(M, N, K, seed=0):
    g = _gen(seed)
    a = torch.randn(M, K, generator=g).half()
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(N, generator=g)).half()
    return a, w, s


def test_dequant_bit_exact(hexmi, oracle):
    a, w, s = _inputs(1, 300, 192, seed=1)
    got = hexmi.dequant_w8(w.cuda(), s.cuda()).cpu().numpy()
    want = oracle.dequant_w8(w.numpy(), s.numpy())
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    # every int8 value with several scales
    allw = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).repeat(4, 1)
    sc = torch.tensor([1.0, 0.25, 0.0123, 0.001], dtype=torch.float16)
    got = hexmi.dequant_w8(allw.cuda(), sc.cuda()).cpu()
    assert torch.equal(got, allw.float() * sc.float()[:, None])


def test_int8_to_fp16_conversion_is_exact(hexmi):
    # A = identity rows pick single weights: C[m, n] = W[n, m] * s[n]; with s = 1 every int8 must come back exactly
    K = 256
    w = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).repeat(48, 1)
    w = torch.stack([w[i].roll(i) for i in range(48)])                  # [48, 256], every value in every column slot
    a = torch.eye(K, dtype=torch.float16)[:64]                           # rows pick k = 0..63
    s = torch.ones(48, dtype=torch.float16)
    c = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    assert torch.equal(c.float(), w[:, :64].t().float())


def test_scale_selection_and_indexing(hexmi, oracle):
    N, K, M = 80, 128, 3
    a = torch.zeros(M, K, dtype=torch.float16)
    a[0, :] = 1.0
    a[1, 7] = 1.0
    a[2, 127] = -2.0
    w = torch.randint(-127, 128, (N, K), generator=_gen(2), dtype=torch.int8)
    s = torch.tensor([2.0 ** -(n % 8) for n in range(N)], dtype=torch.float16)
    c = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu().double()
    sd = s.double()
    assert torch.equal(c[0], (w.double().sum(1) * sd).half().double())
    assert torch.equal(c[1], w[:, 7].double() * sd)
    assert torch.equal(c[2], -2.0 * w[:, 127].double() * sd)
    onehot = torch.zeros(N, dtype=torch.float16)
    onehot[37] = 1.0
    c1 = hexmi.w8a16_matmul(a.cuda(), w.cuda(), onehot.cuda()).cpu()
    assert c1[1, 37] == w[37, 7] and c1[:, :37].abs().sum() == 0 and c1[:, 38:].abs().sum() == 0


@pytest.mark.parametrize("M", [1, 2, 15, 16, 17, 33, 64, 65, 96, 100, 129, 200, 256])
@pytest.mark.parametrize("N,K", [(96, 512), (1000, 256), (16, 64), (11, 4096), (200, 7936)])
def test_w8a16_parity(hexmi, oracle, M, N, K):
    a, w, s = _inputs(M, N, K, seed=3)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)
    assert (got.float() - want.float()).abs().max() / math.sqrt(K) <= 2e-2


@pytest.mark.parametrize("M", [3, 8, 9, 16, 32, 48, 64, 80, 96, 100, 128])
@pytest.mark.parametrize("chunks", [1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 13])
def test_w8a16_every_tail_of_the_chunked_kernel(hexmi, oracle, M, chunks):
    # the chunked kernel (M <= 128) stops copying ahead and lowers its waits by the number of chunks left: every
    # count of chunks up to the depth of the pipeline and beyond, both parities, for every count of row blocks
    K = 256 * chunks
    a, w, s = _inputs(M, 100, K, seed=23 + chunks)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)


@pytest.mark.parametrize("M", [3, 9, 16, 17, 32, 48, 64, 96, 128])
@pytest.mark.parametrize("N", [100, 5000, 10000])
@pytest.mark.parametrize("K", [64, 192, 320, 448, 704, 768, 832, 1536, 1600, 2368, 4096])
def test_w8a16_chunked_kernel_takes_any_k(hexmi, oracle, M, N, K):
    # chunks of 768, 384, 256 or 128 k by the rows and the channel tiles per workgroup (one, two, three at N = 100,
    # 5000, 10000 on 256 CUs), K any multiple of 64: a last chunk that is short, a single short chunk, whole chunks
    a, w, s = _inputs(M, N, K, seed=K + M)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)


@pytest.mark.parametrize("M", [3, 16, 17, 64, 100, 128, 130, 300])
@pytest.mark.parametrize("N", [100, 5000, 10000])
@pytest.mark.parametrize("K", [16, 48, 80, 272, 1008, 1040, 4048])
@pytest.mark.parametrize("zero_points", [False, True])
def test_w8a16_inner_dimension_in_sixteens(hexmi, oracle, M, N, K, zero_points):
    # K a multiple of 16 but not of 64: the chunked kernel masks a lane's sixteen weights past K (its copies are
    # clamped to the row's end); more than 128 rows run it in passes
    if zero_points and (M in (17, 100, 130) or K in (48, 1040)):
        pytest.skip("zero points: a subset of the shapes")
    a, w, s = _inputs(M, N, K, seed=K + M + 1)
    zp = torch.randint(-128, 128, (N,), generator=_gen(K + M), dtype=torch.int8) if zero_points else None
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda(), zero_points=None if zp is None else zp.cuda()).cpu()
    if zp is None:
        want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    else:
        want = torch.from_numpy(oracle.matmul_w8a16_ex(a.numpy(), w.numpy(), s.numpy(), zero_points=zp.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)


@pytest.mark.parametrize("M", [9, 64, 130, 300])
@pytest.mark.parametrize("N", [100, 1000, 1027])
@pytest.mark.parametrize("K", [1, 17, 100, 1001, 4040])
@pytest.mark.parametrize("mode", ["plain", "zero_points", "per_tensor"])
def test_w8a16_unaligned_rows_on_the_matrix_cores(hexmi, oracle, M, N, K, mode):
    # K not a multiple of 16: weight rows start at any byte; more than 8 activation rows run 128x128 tiles whose slabs
    # come through registers (8-byte weight loads at any alignment, guarded bytes at the end of a row)
    a, w, s = _inputs(M, N, K, seed=K + M + N)
    zp = None
    if mode == "zero_points":
        zp = torch.randint(-128, 128, (N,), generator=_gen(K + N), dtype=torch.int8)
    elif mode == "per_tensor":
        s = s[:1].contiguous()
        zp = torch.tensor([-7], dtype=torch.int8)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda(), zero_points=None if zp is None else zp.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16_ex(a.numpy(), w.numpy(), s.numpy(),
                                                   zero_points=None if zp is None else zp.numpy(),
                                                   per_tensor=mode == "per_tensor"))
    assert close16(got, want, max_ulp=1, atol=2e-4)


def test_w8a16_sixteen_wide_tail_ignores_what_lies_behind_the_row(hexmi):
    # K = 784 = 768 + 16: of the last chunk one sixteenth is inside the row; the copies of the rest are clamped to the
    # row's end, where the largest weights and activations sit (their true products are zero)
    M, N, K = 16, 64, 784
    a = torch.zeros(M, K, dtype=torch.float16)
    a[:, -8:] = 60000.0
    a[:, 0] = 1.0
    w = torch.zeros(N, K, dtype=torch.int8)
    w[:, -16:] = 127
    w[:, -8:] = 0
    w[:, 0] = torch.arange(N, dtype=torch.int8)
    s = torch.ones(N, dtype=torch.float16)
    c = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    assert torch.equal(c.float(), torch.arange(N).float().repeat(M, 1))


def test_w8a16_short_last_chunk_ignores_what_lies_behind_the_row(hexmi):
    # K = 832 = 768 + 64: the copies of the last chunk are clamped to the row's end and their units count as zeros,
    # whatever the bytes there are: the largest weights and activations in the last 16 bytes of every row
    M, N, K = 16, 64, 832
    a = torch.zeros(M, K, dtype=torch.float16)
    a[:, -8:] = 60000.0
    a[:, 0] = 1.0
    w = torch.zeros(N, K, dtype=torch.int8)
    w[:, -16:] = 127
    w[:, -8:] = 0                                                        # so the true products of the tail are zero
    w[:, 0] = torch.arange(N, dtype=torch.int8)
    s = torch.ones(N, dtype=torch.float16)
    c = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    assert torch.equal(c.float(), torch.arange(N).float().repeat(M, 1))


@pytest.mark.parametrize("M,N,K", [(4, 14336, 512), (16, 14336, 4096), (9, 28672, 768), (16, 22016, 1024),
                                   (64, 14336, 1024), (128, 22016, 512), (32, 13824, 5120),
                                   # up to 16 rows, two workgroups per CU at a time: one chunk, short last chunks,
                                   # a last workgroup with fewer channels, several rounds
                                   (16, 14336, 256), (3, 13000, 832), (16, 13000, 64), (8, 40000, 640),
                                   (16, 22016, 1984), (5, 52000, 320), (16, 12300, 1280)])
def test_w8a16_more_than_a_workgroup_of_channels_per_cu(hexmi, oracle, M, N, K):
    # N beyond 48 channels per CU: equal workgroups in whole rounds, two at a time per CU with up to 16 rows;
    # the oracle covers every 29th output channel and the first and last 64
    a, w, s = _inputs(M, N, K, seed=N % 97 + M)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    ch = torch.unique(torch.cat([torch.arange(0, N, 29), torch.arange(64), torch.arange(N - 64, N)]))
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w[ch].contiguous().numpy(), s[ch].contiguous().numpy()))
    assert close16(got[:, ch], want, max_ulp=1, atol=2e-4)
    # every output channel, through a permutation of the channels (the order of a sum depends on the workgroup)
    perm = torch.randperm(N, generator=_gen(5))
    got_p = hexmi.w8a16_matmul(a.cuda(), w[perm].contiguous().cuda(), s[perm].contiguous().cuda()).cpu()
    assert close16(got_p, got[:, perm], max_ulp=1, atol=2e-4)


@pytest.mark.parametrize("M", [1, 16, 32, 48, 64, 128, 256])
def test_w8a16_config_sizes(hexmi, oracle, M):
    # measured configuration: N=11008, K=4096; the oracle covers every 43rd output channel, all M rows
    from hexmi.workloads import w8a16_inputs
    inp = w8a16_inputs(M)
    a, w, s = inp["a"], inp["w"], inp["scales"]
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    ch = torch.arange(0, 11008, 43)
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w[ch].contiguous().numpy(), s[ch].contiguous().numpy()))
    assert close16(got[:, ch], want, max_ulp=1, atol=2e-4)
    assert (got[:, ch].float() - want.float()).abs().max() / math.sqrt(4096) <= 2e-2
    # size-independent property over the full output: permuting output channels permutes the columns; bit for bit,
    # except in the chunked kernel (2 < M <= 128), where the workgroup a channel falls in sets the chunk its sum
    # starts with: there to the last place of fp16
    perm = torch.randperm(11008, generator=_gen(9))
    got_p = hexmi.w8a16_matmul(a.cuda(), w[perm].contiguous().cuda(), s[perm].contiguous().cuda()).cpu()
    if M <= 2 or M > 128:
        assert torch.equal(got_p, got[:, perm])
    else:
        assert close16(got_p, got[:, perm], max_ulp=1, atol=2e-4)


@pytest.mark.parametrize("M,N,K", [(300, 520, 192), (130, 264, 320), (2900, 2904, 128), (2100, 4104, 192)])
def test_w8a16_many_rows(hexmi, M, N, K):
    # the tiled kernels (128x128 tiles with four stages, 256x256 with two; odd and even slab counts, ragged edges),
    # checked on sampled rows against a float64 product of the exactly dequantised weights
    a, w, s = _inputs(M, N, K, seed=8)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    rows = torch.cat([torch.arange(0, M, 41), torch.arange(M - 20, M)])
    want = (a[rows].double() @ w.double().t()) * s.double()[None, :]
    assert close16(got[rows], want.half(), max_ulp=1, atol=2e-4)
    assert (got[rows].double() - want).abs().max() / math.sqrt(K) <= 2e-2


def test_w8a16_errors(hexmi):
    a = torch.zeros(2, 64, dtype=torch.float16)
    with pytest.raises(TypeError):
        hexmi.w8a16_matmul(a.float(), torch.zeros(4, 64, dtype=torch.int8), torch.zeros(4, dtype=torch.float16))
    with pytest.raises(ValueError):
        hexmi.w8a16_matmul(a, torch.zeros(4, 32, dtype=torch.int8), torch.zeros(4, dtype=torch.float16))


@pytest.mark.parametrize("M,N,K", [(2, 4, 40), (5, 33, 1), (17, 130, 100), (3, 64, 4100), (70, 20, 72), (4, 32, 128)])
def test_w8a16_any_inner_size(hexmi, oracle, M, N, K):
    # K % 64 != 0 takes the generic kernel: same oracle, same bar
    a, w, s = _inputs(M, N, K, seed=5)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
    assert close16(got, want, max_ulp=1, atol=2e-4)
    # unaligned activations (a view that starts 2 bytes into an allocation) take it too, whatever K is
    buf = torch.zeros(M * K + 1, dtype=torch.float16, device="cuda")
    av = buf[1:].view(M, K)
    av.copy_(a)
    assert torch.equal(hexmi.w8a16_matmul(av, w.cuda(), s.cuda()).cpu(), got)


def test_w8a16_empty_inner_dimension_is_zero(hexmi):
    out = torch.full((3, 8), 7.0, dtype=torch.float16, device="cuda")
    hexmi.w8a16_matmul(torch.zeros(3, 0, dtype=torch.float16, device="cuda"),
                       torch.zeros(8, 0, dtype=torch.int8, device="cuda"),
                       torch.ones(8, dtype=torch.float16, device="cuda"), out=out)
    assert torch.equal(out.cpu(), torch.zeros(3, 8, dtype=torch.float16))


@pytest.mark.parametrize("N,K", [(48, 1024), (1000, 2048), (11008, 4096), (17, 1024)])
def test_pack_w8_bit_exact(hexmi, oracle, N, K):
    w = torch.randint(-128, 128, (N, K), generator=_gen(5), dtype=torch.int8)
    got = hexmi.pack_w8(w.cuda()).cpu().numpy()
    if N * K <= 2 ** 21:
        assert np.array_equal(got, oracle.pack_w8(w.numpy()))
    T = (N + 15) // 16
    padded = torch.zeros(T * 16, K, dtype=torch.int8)
    padded[:N] = w
    want = padded.view(T, 16, K // 64, 4, 16).permute(0, 2, 3, 1, 4).reshape(-1)
    assert np.array_equal(got, want.numpy())


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 40])
@pytest.mark.parametrize("N,K", [(96, 1024), (1000, 2048), (11008, 4096), (11, 4096)])
def test_w8a16_packed_equals_unpacked(hexmi, oracle, M, N, K):
    a, w, s = _inputs(M, N, K, seed=6)
    wp = hexmi.pack_w8(w.cuda())
    got = hexmi.w8a16_matmul_packed(a.cuda(), wp, s.cuda()).cpu()
    if N <= 1000:
        want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.numpy()))
        assert close16(got, want, max_ulp=1, atol=2e-4)
    ref = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    assert close16(got, ref, max_ulp=1, atol=2e-4)            # other kernels sum in another order
    with pytest.raises(ValueError):
        hexmi.w8a16_matmul_packed(a.cuda(), wp[:-16], s.cuda())


def test_packed_weights_through_a_tensor_file(hexmi, tmp_path):
    # pre-packed weights kept in the reference's raw tensor format (test/utils/dsp/include/tensor.h:235-260)
    a, w, s = _inputs(8, 1000, 2048, seed=7)
    wp = hexmi.pack_w8(w.cuda())
    path = str(tmp_path / "wp.bin")
    hexmi.save_tensor(path, wp)
    back = hexmi.load_tensor(path)
    assert back.dtype == torch.int8 and torch.equal(back, wp.cpu())
    got = hexmi.w8a16_matmul_packed(a.cuda(), back.cuda(), s.cuda()).cpu()
    assert torch.equal(got, hexmi.w8a16_matmul_packed(a.cuda(), wp, s.cuda()).cpu())


# ---- the (channel range x K part) kernel behind hexmi_gemm_w8a16_ws -------------------------------------------

def _ws_call(hexmi, a, w, s, ws, ws_bytes=None):
    """hexmi_gemm_w8a16_ws through the C ABI on device tensors; ws may be None."""
    lib = hexmi.lib()
    M, K = a.shape
    N = w.shape[0]
    c = torch.full((M, N), 7.0, dtype=torch.float16, device="cuda")
    rc = lib.hexmi_gemm_w8a16_ws(M, N, K, a.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(),
                                 ws.data_ptr() if ws is not None else None,
                                 (ws.numel() if ws is not None else 0) if ws_bytes is None else ws_bytes,
                                 torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return rc, c


# shapes the library gives to that kernel: many channels per CU, a long K, or few 128 x 128 tiles; K parts 1, 2, 8;
# ragged channel ranges, a last row tile of one row, a last channel range of eight channels
SPLIT_SHAPES = [(64, 96, 8192), (33, 12300, 128), (256, 1000, 1024), (129, 2000, 384), (200, 8192, 2048),
                (100, 13000, 256), (80, 264, 16384), (250, 72, 4096)]


@pytest.mark.parametrize("M,N,K", SPLIT_SHAPES)
def test_w8a16_split_parity(hexmi, oracle, M, N, K):
    a, w, s = _inputs(M, N, K, seed=11)
    ad, wd, sd = a.cuda(), w.cuda(), s.cuda()
    need = hexmi.lib().hexmi_gemm_w8a16_workspace(M, N, K)
    # the scratch starts out as garbage: the library must not rely on its contents
    ws = torch.full((max(need, 16),), 0xA5, dtype=torch.uint8, device="cuda")
    rc, got = _ws_call(hexmi, ad, wd, sd, ws)
    assert rc == 0
    ch = torch.arange(0, N, max(1, N // 160))
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w[ch].contiguous().numpy(), s[ch].contiguous().numpy()))
    assert close16(got.cpu()[:, ch], want, max_ulp=1, atol=2e-4)
    assert (got.cpu()[:, ch].float() - want.float()).abs().max() / math.sqrt(K) <= 2e-2
    # the operator front takes the same path (it keeps a workspace per stream) and gives the same bits, again and again
    for _ in range(3):
        assert torch.equal(hexmi.w8a16_matmul(ad, wd, sd), got)
    # against the kernels of the plain entry point (another summation order; each is within one unit in the last
    # place of the oracle, so of each other within two; where the value is a cancellation residue of fp32 partial sums
    # the two orders differ by the rounding of those sums, which grows with K)
    plain = torch.empty_like(got)
    assert hexmi.lib().hexmi_gemm_w8a16(M, N, K, ad.data_ptr(), wd.data_ptr(), sd.data_ptr(), plain.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert close16(got.cpu(), plain.cpu(), max_ulp=2, atol=2e-4 * max(1.0, K / 4096))
    # permuting output channels permutes the columns, bit for bit
    perm = torch.randperm(N, generator=_gen(12))
    rc, got_p = _ws_call(hexmi, ad, w[perm].contiguous().cuda(), s[perm].contiguous().cuda(), ws)
    assert rc == 0 and torch.equal(got_p.cpu(), got.cpu()[:, perm])


@pytest.mark.parametrize("M", [64, 128, 256])
def test_w8a16_down_projection_sizes(hexmi, oracle, M):
    # the other projection of the benchmark's model: N = 4096, K = 11008 (the oracle on every 29th channel)
    N, K = 4096, 11008
    a, w, s = _inputs(M, N, K, seed=13)
    assert hexmi.lib().hexmi_gemm_w8a16_workspace(M, N, K) > 0
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    ch = torch.arange(0, N, 29)
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w[ch].contiguous().numpy(), s[ch].contiguous().numpy()))
    assert close16(got[:, ch], want, max_ulp=1, atol=2e-4)
    assert (got[:, ch].float() - want.float()).abs().max() / math.sqrt(K) <= 2e-2
    perm = torch.randperm(N, generator=_gen(14))
    got_p = hexmi.w8a16_matmul(a.cuda(), w[perm].contiguous().cuda(), s[perm].contiguous().cuda()).cpu()
    assert torch.equal(got_p, got[:, perm])


@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("N,K", [(4096, 11008), (100, 80), (37, 16384), (64, 1040), (9, 5120)])
def test_w8a16_decode_any_row_length(hexmi, oracle, M, N, K):
    # one or two rows with K % 16 == 0 outside {1024, 2048, 4096, 8192}: the masked form of the decode kernel (the
    # chunked kernel for two rows of 11008)
    a, w, s = _inputs(M, N, K, seed=15)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
    ch = torch.arange(0, N, max(1, N // 200))
    want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w[ch].contiguous().numpy(), s[ch].contiguous().numpy()))
    assert close16(got[:, ch], want, max_ulp=1, atol=2e-4)
    perm = torch.randperm(N, generator=_gen(16))
    got_p = hexmi.w8a16_matmul(a.cuda(), w[perm].contiguous().cuda(), s[perm].contiguous().cuda()).cpu()
    if M == 2 and K >= 8192 and N >= 4096:
        # two rows over a long K run the chunked kernel, where the owning workgroup sets the chunk a sum starts with
        assert close16(got_p, got[:, perm], max_ulp=1, atol=2e-4)
    else:
        assert torch.equal(got_p, got[:, perm])


def test_w8a16_workspace_contract(hexmi):
    lib = hexmi.lib()
    # shapes the plain kernels keep: no workspace asked for, and a NULL workspace is fine
    assert lib.hexmi_gemm_w8a16_workspace(16, 11008, 4096) == 0
    assert lib.hexmi_gemm_w8a16_workspace(64, 11008, 4096) == 0
    assert lib.hexmi_gemm_w8a16_workspace(0, 64, 64) == 0
    M, N, K = 64, 4096, 11008
    need = lib.hexmi_gemm_w8a16_workspace(M, N, K)
    assert need > 0
    a, w, s = _inputs(M, N, K, seed=17)
    ad, wd, sd = a.cuda(), w.cuda(), s.cuda()
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ws.fill_(0xA5)                                            # garbage: the library clears what it needs
    rc, with_ws = _ws_call(hexmi, ad, wd, sd, ws)
    assert rc == 0
    # word 0 is the guard's error word (no bounded wait expired); the flags behind it are back to zero for the next call
    header = ws[:1024].view(torch.int32).cpu()
    assert header[0].item() == 0 and int(header[:64].abs().sum()) == 0
    rc, _ = _ws_call(hexmi, ad, wd, sd, ws, ws_bytes=need - 1)
    assert rc == hexmi._lib.EINVAL
    rc, no_ws = _ws_call(hexmi, ad, wd, sd, None)             # the plain kernels
    assert rc == 0 and close16(no_ws.cpu(), with_ws.cpu(), max_ulp=2, atol=2e-4)
    rc, _ = _ws_call(hexmi, ad, wd, sd, ws, ws_bytes=-1)
    assert rc == hexmi._lib.EINVAL


# ---- quant.dcast with a zero point, per channel or per tensor ------------------------------------------------------

@pytest.mark.parametrize("per_tensor", [False, True])
def test_dequant_with_zero_point_bit_exact(hexmi, oracle, per_tensor):
    g = _gen(18)
    w = torch.randint(-128, 128, (300, 192), generator=g, dtype=torch.int8)
    n = 1 if per_tensor else 300
    s = (0.001 + 0.019 * torch.rand(n, generator=g)).half()
    zp = torch.randint(-128, 128, (n,), generator=g, dtype=torch.int8)
    got = hexmi.dequant_w8(w.cuda(), s.cuda(), zero_points=zp.cuda()).cpu().numpy()
    want = oracle.dequant_w8_ex(w.numpy(), s.numpy(), zp.numpy(), per_tensor)
    assert (got.view(np.uint32) == want.view(np.uint32)).all()
    # every (weight, zero point) pair of int8 with scale 1: the integer difference, exactly
    allw = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).repeat(256, 1)
    allz = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8)
    got = hexmi.dequant_w8(allw.cuda(), torch.ones(256, dtype=torch.float16).cuda(), zero_points=allz.cuda()).cpu()
    assert torch.equal(got, allw.float() - allz.float()[:, None])
    # without a zero point and per channel it is the symmetric entry point
    s2 = (0.001 + 0.019 * torch.rand(300, generator=g)).half()
    assert torch.equal(hexmi.dequant_w8(w.cuda(), s2.cuda()).cpu(), w.float() * s2.float()[:, None])


@pytest.mark.parametrize("per_tensor", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 96, 512), (16, 1000, 256), (70, 130, 128), (33, 40, 4096), (5, 33, 100),
                                   (3, 64, 72),
                                   # the decode kernels and every form of the chunked kernel (chunks of 768, 384, 256
                                   # and 128 k, short last chunks, two workgroups per CU), which subtract the zero
                                   # point in registers
                                   (1, 500, 4096), (2, 300, 2048), (1, 200, 11008), (2, 4100, 8192), (4, 100, 832),
                                   (16, 5000, 1536), (9, 10000, 4096), (32, 5000, 832), (48, 100, 768),
                                   (64, 10000, 1024), (96, 100, 512), (128, 5000, 256), (16, 14336, 512),
                                   (200, 136, 256), (300, 1000, 832)])
def test_w8a16_with_zero_point_parity(hexmi, oracle, per_tensor, M, N, K):
    g = _gen(19)
    a = torch.randn(M, K, generator=g).half()
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    n = 1 if per_tensor else N
    s = (0.001 + 0.019 * torch.rand(n, generator=g)).half()
    zp = torch.randint(-128, 128, (n,), generator=g, dtype=torch.int8)
    got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda(), zero_points=zp.cuda()).cpu()
    want = torch.from_numpy(oracle.matmul_w8a16_ex(a.numpy(), w.numpy(), s.numpy(), zp.numpy(), per_tensor))
    assert close16(got, want, max_ulp=1, atol=4e-4)
    # zero point selection is exact: activations that pick one weight give (w - zp) * s with s a power of two
    sel = torch.zeros(1, K, dtype=torch.float16)
    sel[0, K - 1] = 1.0
    s2 = torch.tensor([2.0 ** -(i % 6) for i in range(n)], dtype=torch.float16)
    got = hexmi.w8a16_matmul(sel.cuda(), w.cuda(), s2.cuda(), zero_points=zp.cuda()).cpu().double()
    zd = zp.double().expand(N) if per_tensor else zp.double()
    sd = s2.double().expand(N) if per_tensor else s2.double()
    assert torch.equal(got[0], (w[:, K - 1].double() - zd) * sd)
    # per-tensor scale without a zero point
    if per_tensor:
        got = hexmi.w8a16_matmul(a.cuda(), w.cuda(), s.cuda()).cpu()
        want = torch.from_numpy(oracle.matmul_w8a16(a.numpy(), w.numpy(), s.expand(N).contiguous().numpy()))
        assert close16(got, want, max_ulp=1, atol=2e-4)
