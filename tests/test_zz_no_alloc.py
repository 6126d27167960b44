"""The entry point that allocates nothing (hexmi_block_sum_static) against the workspace entry point it mirrors
(hexmi_block_sum_ws), through the C ABI: bit-exact, on two calls in a row, the second with a smaller input (the
library's fixed scratch array keeps the first call's partial sums)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _both(lib, _lib, x, n, block, code):
    programs = (n + block - 1) // block
    need = lib.hexmi_block_sum_workspace(n, block, code)
    ws = torch.empty(max(need, 4), dtype=torch.uint8, device="cuda")
    want = torch.zeros(programs, dtype=x.dtype, device="cuda")
    got = torch.full((programs,), 7.0, dtype=x.dtype, device="cuda")
    assert lib.hexmi_block_sum_ws(x.data_ptr(), want.data_ptr(), n, block, code, ws.data_ptr(), need, None) == _lib.OK
    # The first launch of a kernel in a process makes the HIP runtime load its code object (device memory the runtime
    # owns), and the first call on a device looks up the scratch array: one call goes ahead of the measured one.
    assert lib.hexmi_block_sum_static(x.data_ptr(), got.data_ptr(), n, block, code, None) == _lib.OK
    got.fill_(7.0)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]                 # hipMemGetInfo: sees every allocation on the device,
    assert lib.hexmi_block_sum_static(x.data_ptr(), got.data_ptr(), n, block, code, None) == _lib.OK
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before             # torch's own allocator included
    assert torch.cuda.mem_get_info()[0] == free_before
    return got.cpu(), want.cpu(), need


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_static_block_sum_matches_workspace_entry(hexmi, dtype):
    from hexmi import _lib
    lib = _lib.lib()
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[dtype]
    x = torch.randn(3 << 20, generator=_gen(7)).to(dtype).cuda()
    # first call: 3 programs of 2^20 elements (768 partial sums in the scratch)
    got, want, need = _both(lib, _lib, x, 3 << 20, 1 << 20, code)
    assert need == 768 * 4
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    ref = x.double().view(3, -1).sum(1).cpu()
    assert (got.double() - ref).abs().max() <= (1e-2 if dtype == torch.float32 else 4.1)
    # second call, smaller input on another part of the data: one program of 300001 elements (74 partial sums, the
    # last run ragged); the scratch still holds the first call's 768
    y = x[12345:12345 + 300001]
    got2, want2, need2 = _both(lib, _lib, y, 300001, 300001, code)
    assert need2 == 74 * 4
    assert torch.equal(got2.view(torch.uint8), want2.view(torch.uint8))
    assert abs(got2.double().item() - y.double().sum().item()) <= (1e-2 if dtype == torch.float32 else 2.1)
    # a shape that needs no scratch (small programs) goes through as well
    got3, want3, need3 = _both(lib, _lib, x, 100000, 1000, code)
    assert need3 == 0 and torch.equal(got3.view(torch.uint8), want3.view(torch.uint8))


def test_static_block_sum_limits(hexmi):
    from hexmi import _lib
    lib = _lib.lib()
    assert lib.hexmi_block_sum_static_max_n() == 1 << 30
    x = torch.zeros(16, device="cuda")
    # beyond the fixed capacity: refused before anything is read
    assert lib.hexmi_block_sum_static(x.data_ptr(), x.data_ptr(), (1 << 30) + 1, 1 << 20, _lib.F32, None) == _lib.ETOOBIG
    assert lib.hexmi_block_sum_static(None, None, 4, 4, _lib.F32, None) == _lib.EINVAL
    assert lib.hexmi_block_sum_static(None, None, 0, 4, _lib.F32, None) == _lib.OK


def test_static_block_sum_under_graph_capture(hexmi):
    # the callers this entry point is for: code under HIP graph capture. Captured after one warm-up call (the first
    # call on a device looks up the scratch array's address), replayed on changing inputs with eager work between.
    from hexmi import _lib
    lib = _lib.lib()
    n, block = 1 << 21, 1 << 20
    g = _gen(8)
    x = torch.randn(n, generator=g).cuda()
    out = torch.zeros(2, device="cuda")
    eager = torch.zeros(2, device="cuda")
    assert lib.hexmi_block_sum_static(x.data_ptr(), eager.data_ptr(), n, block, _lib.F32, None) == _lib.OK
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            assert lib.hexmi_block_sum_static(x.data_ptr(), out.data_ptr(), n, block, _lib.F32, stream.cuda_stream) == _lib.OK
    for replay in range(3):
        x.copy_((torch.randn(n, generator=g) * (1 + replay)).cuda())
        assert lib.hexmi_block_sum_static(x.data_ptr(), eager.data_ptr(), n, block, _lib.F32, None) == _lib.OK
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), replay
