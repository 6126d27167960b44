"""Compiled C++ programs call the C ABI (tests/c_abi/*.cpp, built against include/hexmi.h and linked with
libhexmi.so) in the shape of the reference's device wrappers: they read raw tensor files, run one operator, check
it with a scalar loop and the wrapper's own MAX_DIFF, write the result as a raw tensor file and report through the
exit status. The files are written and read back here with hexmi/tensor_file.py, so the format is exercised across
the language boundary, and the result is checked a second time against the oracle."""
import importlib.util
import os
import subprocess

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def _binaries():
    spec = importlib.util.spec_from_file_location("c_abi_build", os.path.join(HERE, "c_abi", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    paths = {n: mod.binary(n) for n in mod.PROGRAMS}
    if not all(os.path.exists(p) for p in paths.values()):
        mod.build()                                        # normally built beforehand by __graft_entry__.build()
    return paths


def _wrapper_inputs(shape, seed):
    # set_pointer_random of the wrappers: N(0, 0.5) rounded to four decimals, then to fp16
    g = torch.Generator().manual_seed(seed)
    return (torch.round(torch.randn(*shape, generator=g) * 0.5 * 10000) / 10000).half()


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=100)
    return r.returncode, r.stdout + r.stderr


def test_matmul_caller(hexmi, oracle, tmp_path):
    # test/python/mlir/hexkl_linalg_matmul/wrapper.cpp:31-81: N = 1024 rows, K = 64, M = 512 columns, MAX_DIFF 1e-2
    act, w = _wrapper_inputs((1024, 64), 31), _wrapper_inputs((64, 512), 32)
    paths = [str(tmp_path / n) for n in ("act.bin", "w.bin", "out.bin")]
    hexmi.save_tensor(paths[0], act)
    hexmi.save_tensor(paths[1], w)
    rc, log = _run([_binaries()["matmul_caller"]] + paths)
    assert rc == 0, log
    assert "Pass" in log and "hexmi " in log
    out = hexmi.load_tensor(paths[2])
    assert out.dtype == torch.float32 and tuple(out.shape) == (1024, 512)
    want = torch.from_numpy(oracle.matmul(act.numpy(), w.numpy(), out_dtype=np.float32))
    assert torch.allclose(out, want, rtol=1e-5, atol=1e-5)
    # the same call from Python gives the same bits
    got = hexmi.matmul(act.cuda(), w.cuda(), out_dtype=torch.float32).cpu()
    assert torch.equal(got, out)


def test_attention_caller(hexmi, oracle, tmp_path):
    # test/python/mlir/hexkl_attention/wrapper.cpp:151-221: Z = H = 1, N_CTX = 1024, D_HEAD = 64, scale 0.5,
    # fp16 Q / K / V, fp32 output, MAX_DIFF 1e-3
    q, k, v = (_wrapper_inputs((1, 1, 1024, 64), s) for s in (33, 34, 35))
    paths = [str(tmp_path / n) for n in ("q.bin", "k.bin", "v.bin", "out.bin")]
    for p, t in zip(paths, (q, k, v)):
        hexmi.save_tensor(p, t)
    rc, log = _run([_binaries()["attention_caller"]] + paths)
    assert rc == 0, log
    assert "Pass" in log
    out = hexmi.load_tensor(paths[3])
    assert out.dtype == torch.float32 and tuple(out.shape) == (1, 1, 1024, 64)
    want = torch.from_numpy(oracle.attention(q.numpy(), k.numpy(), v.numpy(), 0.5, False, out_dtype=np.float32))
    assert (out - want).abs().max() <= 1e-3
    got = hexmi.flash_attention(q.cuda(), k.cuda(), v.cuda(), 0.5, False, out_dtype=torch.float32).cpu()
    assert torch.equal(got, out)


def test_callers_report_bad_input_through_the_exit_status(hexmi, tmp_path):
    bad = str(tmp_path / "bad.bin")
    hexmi.save_tensor(bad, torch.zeros(4, 4))              # fp32 where fp16 is expected
    rc, log = _run([_binaries()["matmul_caller"], bad, bad, str(tmp_path / "o.bin")])
    assert rc == 2 and "expected fp16" in log
