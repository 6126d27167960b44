"""The measurement probes of include/hexmi_calibrate.h (hexmi_mfma_peak, hexmi_issue_slots, hexmi_lds_read_pattern):
argument checks and that every case launches and runs to completion. What they measure (time ratios between cases)
depends on the box's clocks and is recorded by bench.py, not asserted here."""
import pytest
import torch

from hexmi import _lib

pytestmark = pytest.mark.gpu


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


def test_issue_slots_every_case_runs():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 512, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for shape in (0, 1):
        for kind in (0, 1, 2, 3, 4):
            for per in (0, 2, 5, 8):
                _lib.check(lib.hexmi_issue_slots(shape, kind, per, 100, 2, sink.data_ptr(), st), "hexmi_issue_slots")
    torch.cuda.synchronize()


def test_lds_patterns_every_case_runs():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for p in range(7):
        _lib.check(lib.hexmi_lds_read_pattern(p, 200, sink.data_ptr(), st), "hexmi_lds_read_pattern")
    torch.cuda.synchronize()


def test_launches_are_bounded():
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 1024, device="cuda")
    ops = torch.zeros(1024, dtype=torch.float16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    too_many = (1 << 20) + 1
    assert lib.hexmi_mfma_peak(0, _lib.F16, ops.data_ptr(), too_many, 1, sink.data_ptr(), st) == _lib.ETOOBIG
    assert lib.hexmi_issue_slots(0, 0, 0, too_many, 1, sink.data_ptr(), st) == _lib.ETOOBIG
    assert lib.hexmi_lds_read_pattern(0, too_many, sink.data_ptr(), st) == _lib.ETOOBIG


def test_l2_stream_runs_and_is_bounded():
    lib = _lib.lib()
    cus = lib.hexmi_num_cus()
    sink = torch.empty(cus * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    region = 64 << 10
    own = torch.zeros(region * cus, dtype=torch.uint8, device="cuda")
    for to_lds in (0, 1):
        for shared in (0, 1):
            assert lib.hexmi_l2_stream(to_lds, shared, region, 4, own.data_ptr(), sink.data_ptr(), st) == _lib.OK
    torch.cuda.synchronize()
    assert lib.hexmi_l2_stream(1, 1, region + 1024, 4, own.data_ptr(), sink.data_ptr(), st) == _lib.EINVAL
    assert lib.hexmi_l2_stream(1, 1, region, -1, own.data_ptr(), sink.data_ptr(), st) == _lib.EINVAL
    assert lib.hexmi_l2_stream(1, 1, region, 1, None, sink.data_ptr(), st) == _lib.EINVAL
    assert lib.hexmi_l2_stream(1, 1, region, (1 << 20) + 1, own.data_ptr(), sink.data_ptr(), st) == _lib.ETOOBIG
    assert lib.hexmi_l2_stream(1, 1, 1 << 30, 1 << 10, own.data_ptr(), sink.data_ptr(), st) == _lib.ETOOBIG
