"""The measurement aids of the C ABI (hexmi_mfma_peak, hexmi_issue_slots, hexmi_lds_read_pattern): argument checks,
and that each launch runs to completion and orders its cases the way the kernels' design assumes."""
import pytest
import torch

from hexmi import _lib

pytestmark = pytest.mark.gpu


def _ms(fn):
    # the fastest of five after three untimed launches: these tests compare times of launches made one after the
    # other, and the first launches on an idle GPU run at a lower clock
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1))
    return best


def test_argument_checks():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    assert lib.hexmi_issue_slots(2, 0, 0, 10, 1, sink.data_ptr(), st) == _lib.EINVAL       # shape
    assert lib.hexmi_issue_slots(0, 5, 0, 10, 1, sink.data_ptr(), st) == _lib.EINVAL       # kind
    assert lib.hexmi_issue_slots(0, 0, 7, 10, 1, sink.data_ptr(), st) == _lib.EINVAL       # per_mfma not offered
    assert lib.hexmi_issue_slots(0, 0, 0, 10, 3, sink.data_ptr(), st) == _lib.EINVAL       # waves per SIMD
    assert lib.hexmi_issue_slots(0, 0, 0, 10, 1, None, st) == _lib.EINVAL
    assert lib.hexmi_lds_read_pattern(7, 10, sink.data_ptr(), st) == _lib.EINVAL
    assert lib.hexmi_lds_read_pattern(0, -1, sink.data_ptr(), st) == _lib.EINVAL
    assert lib.hexmi_lds_read_pattern(0, 10, None, st) == _lib.EINVAL


def test_mfma_peak_runs_both_shapes():
    lib = _lib.lib()
    ops = torch.zeros(1024, dtype=torch.float16, device="cuda")
    sink = torch.empty(lib.hexmi_num_cus() * 512, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for shape in (0, 1):
        for code in (_lib.F16, _lib.BF16):
            _lib.check(lib.hexmi_mfma_peak(shape, code, ops.data_ptr(), 100, 2, sink.data_ptr(), st), "hexmi_mfma_peak")
    torch.cuda.synchronize()
    assert float(sink.abs().max()) == 0.0                  # zero operands: every accumulator stays zero


def test_issue_slots_vector_work_beyond_the_shadow_costs_time():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 512, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    t = {}
    for per in (0, 2, 8):
        t[per] = _ms(lambda: _lib.check(lib.hexmi_issue_slots(1, 0, per, 2000, 1, sink.data_ptr(), st), "hexmi_issue_slots"))
    # two vector instructions per 16x16x32 MFMA ride along (measured +5 %), eight more than double the time
    assert t[2] < 1.3 * t[0]
    assert t[8] > 1.7 * t[0]
    for shape in (0, 1):
        for kind in (0, 1, 2, 3, 4):
            _lib.check(lib.hexmi_issue_slots(shape, kind, 5, 100, 2, sink.data_ptr(), st), "hexmi_issue_slots")
    torch.cuda.synchronize()


def test_lds_patterns_swizzles_in_use_read_at_the_linear_rate():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    t = [_ms(lambda: _lib.check(lib.hexmi_lds_read_pattern(p, 2000, sink.data_ptr(), st), "hexmi_lds_read_pattern"))
         for p in range(7)]
    for p in (1, 3, 5):                                    # the patterns the kernels use
        assert t[p] < 1.25 * t[0], (p, t)
    for p in (2, 4):                                       # the ones they replaced: measured 1.75x
        assert t[p] > 1.4 * t[0], (p, t)
    assert t[6] > 2.0 * t[0], t                            # no swizzle at all: measured 3.5x
