"""The C-ABI library loads without a GPU and exports every symbol include/hexmi.h declares; the Python
loader binds exactly that set; argument checks that need no device return the documented status."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hexmi.h")
PROBE_HEADER = os.path.join(ROOT, "include", "hexmi_calibrate.h")     # measurement probes, not the operator ABI


def _declared(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hexmi_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = _declared()
    for must in ("hexmi_softmax", "hexmi_rms_norm", "hexmi_layer_norm", "hexmi_matmul_f16f16_f32", "hexmi_gemm",
                 "hexmi_gemm_w8a16", "hexmi_dequant_w8", "hexmi_flash_attn_fwd", "hexmi_attention", "hexmi_unary",
                 "hexmi_binary", "hexmi_block_sum", "hexmi_rope", "hexmi_pack_w8", "hexmi_gemm_w8a16_packed"):
        assert must in names


def test_library_exports_every_declared_symbol():
    import hexmi
    assert os.path.exists(hexmi.LIB_PATH), "build libhexmi.so first: python hexagon-mlir_amd/build.py"
    handle = ctypes.CDLL(hexmi.LIB_PATH)
    for name in _declared() + _declared(PROBE_HEADER):
        assert hasattr(handle, name), "libhexmi.so does not export %s" % name


def test_loader_binds_exactly_the_header():
    from hexmi import _lib
    assert sorted(_lib.SIGNATURES) == _declared()
    assert sorted(_lib.PROBE_SIGNATURES) == _declared(PROBE_HEADER)
    assert not set(_lib.SIGNATURES) & set(_lib.PROBE_SIGNATURES)      # the operator header declares no probe
    lib = _lib.lib()
    assert lib.hexmi_version().decode().startswith("hexmi ")
    assert "invalid" in _lib.strerror(_lib.EINVAL)


def test_argument_errors_need_no_device():
    from hexmi import _lib
    lib = _lib.lib()
    # negative sizes and short leading dimensions are rejected before any HIP call
    assert lib.hexmi_softmax(None, None, -1, 8, 8, 8, _lib.F32, None) == _lib.EINVAL
    assert lib.hexmi_softmax(None, None, 4, 8, 4, 8, _lib.F32, None) == _lib.EINVAL
    assert lib.hexmi_softmax(None, None, 4, 8, 8, 8, _lib.F32, None) == _lib.EINVAL      # null pointers
    assert lib.hexmi_softmax(None, None, 0, 8, 8, 8, _lib.F32, None) == _lib.OK          # empty: nothing to do
    assert lib.hexmi_rms_norm(None, None, None, 3, 5, 1e-5, _lib.F16, None) == _lib.EINVAL
    assert lib.hexmi_layer_norm(None, None, None, None, None, None, 0, 0, 1e-5, _lib.F16, None) == _lib.OK


def test_missing_library_fails_loudly(monkeypatch):
    from hexmi import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libhexmi.so")
    with pytest.raises(RuntimeError, match="no CPU or eager fallback"):
        _lib.lib()


def test_ops_refuse_to_run_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    import hexmi
    with pytest.raises(RuntimeError, match="needs a GPU"):
        hexmi.softmax(torch.zeros(2, 2))


def test_kernel_front_checks_grid_and_options():
    import torch
    import hexmi
    k = hexmi.kernels.softmax_kernel
    with pytest.raises(ValueError, match="at least 1 thread"):
        k[(0,)]
    x = torch.zeros(2, 2)
    with pytest.raises(TypeError):
        k[(1,)](x, x, NUM_ROWS=2, NUM_COLS=2, BLOCK_SIZE=2, notAnOption=True)
    with pytest.raises(RuntimeError, match="outside"):
        k(x, x)


def test_dtype_ids_are_the_reference_tensor_ids():
    # enum DataType of the reference's test/utils/dsp/include/tensor.h:26-38: Half = 1, Float = 2, Int8 = 4;
    # bfloat16 has no id there and sits outside the table (0..10)
    from hexmi import _lib, tensor_file
    text = open(HEADER).read()
    ids = dict((k, int(v)) for k, v in re.findall(r"(HEXMI_(?:F16|F32|I8|BF16))\s*=\s*(\d+)", text))
    assert ids == {"HEXMI_F16": 1, "HEXMI_F32": 2, "HEXMI_I8": 4, "HEXMI_BF16": 16}
    assert (_lib.F16, _lib.F32, _lib.I8, _lib.BF16) == (1, 2, 4, 16)
    import numpy as np
    for code, np_type in ((_lib.F16, np.float16), (_lib.F32, np.float32), (_lib.I8, np.int8)):
        assert tensor_file._ID_TO_NP[code] is np_type
    assert _lib.BF16 not in tensor_file._ID_TO_NP


def test_block_sum_workspace_query_needs_no_device():
    from hexmi import _lib
    lib = _lib.lib()
    assert lib.hexmi_block_sum_workspace(1 << 20, 1 << 20, _lib.F16) == 256 * 4       # one program: two passes
    assert lib.hexmi_block_sum_workspace(1 << 20, 4096, _lib.F32) == 0                # small programs: one pass
    assert lib.hexmi_block_sum_workspace(300000, 131072, _lib.F32) == 74 * 4
    assert lib.hexmi_block_sum_workspace(300000, 100000, _lib.F32) == 0               # runs would straddle programs
    assert lib.hexmi_block_sum_workspace(0, 16, _lib.F32) == 0
    assert lib.hexmi_block_sum_ws(None, None, -1, 4, _lib.F32, None, 0, None) == _lib.EINVAL
    assert "capacity" in _lib.strerror(_lib.ETOOBIG)


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
