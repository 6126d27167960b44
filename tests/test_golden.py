"""The committed vectors of tests/golden/fixtures.npz (made by tests/golden/make_fixtures.py from PyTorch CPU calls
in float64) against the CPU oracle (no GPU) and against the HIP kernels (-m gpu). Tolerances: fp32 results 1e-5
relative to the largest expected value; results rounded to fp16 one unit in the last place of the expectation
(2^-10 relative) plus the rounding of intermediate fp32 sums."""
import math
import os

import numpy as np
import pytest
import torch

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.npz"), allow_pickle=False)


def T(name):
    return torch.from_numpy(FIX[name])


def close32(got, want, rel=1e-5):
    got, want = torch.as_tensor(got).double(), want.double()
    return bool(((got - want).abs() <= rel * want.abs().max() + 1e-30).all())


def close_half(got, want, extra=0.0):
    got, want = torch.as_tensor(got).double(), want.double()
    return bool(((got - want).abs() <= 2.0 ** -10 * want.abs() + extra + 1e-7).all())


# ---- CPU: the oracle reproduces the stored expectations -----------------------------------------------------------
def test_oracle_rows(oracle):
    assert close32(oracle.softmax(FIX["softmax_x"]), T("softmax_y"))
    x, w, b = FIX["norm_x"], FIX["norm_w"], FIX["norm_b"]
    assert close_half(oracle.rms_norm(x, w, 1e-5), T("rms_y"))
    y, mean, rstd = oracle.layer_norm(x, w, b, 1e-5)
    assert close_half(y, T("ln_y"), extra=1e-3) and close32(mean, T("ln_mean"), 1e-5) and close32(rstd, T("ln_rstd"), 1e-5)


def test_oracle_matmuls(oracle):
    a, b = FIX["mm_a"], FIX["mm_b"]
    assert close32(oracle.matmul(a, b, out_dtype=np.float32), T("mm_c"))
    assert close32(oracle.matmul(a, np.ascontiguousarray(b.T), out_dtype=np.float32, trans_b=True), T("mm_c"))
    assert close_half(oracle.matmul(a, b), T("mm_c"), extra=1e-5)
    assert close_half(oracle.matmul_w8a16(FIX["w8_a"], FIX["w8_w"], FIX["w8_s"]), T("w8_c"), extra=1e-5)


def test_oracle_attention(oracle):
    q, k, v = FIX["fa_q"], FIX["fa_k"], FIX["fa_v"]
    assert close32(oracle.attention(q, k, v, 1 / 8, False, out_dtype=np.float32), T("fa_o"), 1e-5)
    assert close32(oracle.attention(q, k, v, 1 / 8, True, out_dtype=np.float32), T("fa_o_causal"), 1e-5)
    got = oracle.attention_masked(FIX["ma_q"], FIX["ma_k"], FIX["ma_v"], FIX["ma_mask"], 1 / 8, out_dtype=np.float32)
    assert close32(got, T("ma_o"), 1e-5)


def test_oracle_elementwise(oracle):
    x = FIX["ew_x"]
    assert close_half(oracle.unary("gelu_tanh", x), T("gelu_y"), extra=1e-6)
    assert close_half(oracle.unary("silu", x), T("silu_y"), extra=1e-6)
    assert close_half(oracle.rope(FIX["rope_x"], 10000.0), T("rope_y"), extra=1e-6)
    assert close32(oracle.block_sum(FIX["sum_x"], 32), T("sum_y"), 1e-6)


# ---- GPU: the HIP kernels reproduce the stored expectations -------------------------------------------------------
@pytest.mark.gpu
def test_hip_rows(hexmi):
    assert close32(hexmi.softmax(T("softmax_x").cuda()).cpu(), T("softmax_y"))
    x, w, b = T("norm_x").cuda(), T("norm_w").cuda(), T("norm_b").cuda()
    assert close_half(hexmi.rms_norm(x, w, 1e-5).cpu(), T("rms_y"))
    mean = torch.empty(x.shape[0], device="cuda")
    rstd = torch.empty(x.shape[0], device="cuda")
    y = hexmi.layer_norm(x, w, b, 1e-5, mean=mean, rstd=rstd)
    assert close_half(y.cpu(), T("ln_y"), extra=1e-3)
    assert close32(mean.cpu(), T("ln_mean"), 1e-5) and close32(rstd.cpu(), T("ln_rstd"), 1e-5)


@pytest.mark.gpu
def test_hip_matmuls(hexmi):
    a, b = T("mm_a").cuda(), T("mm_b").cuda()
    assert close32(hexmi.matmul(a, b, out_dtype=torch.float32).cpu(), T("mm_c"))
    assert close32(hexmi.matmul(a, b.t().contiguous(), out_dtype=torch.float32, trans_b=True).cpu(), T("mm_c"))
    assert close_half(hexmi.matmul(a, b).cpu(), T("mm_c"), extra=1e-5)
    got = hexmi.w8a16_matmul(T("w8_a").cuda(), T("w8_w").cuda(), T("w8_s").cuda()).cpu()
    assert close_half(got, T("w8_c"), extra=1e-5)


@pytest.mark.gpu
def test_hip_attention(hexmi):
    q, k, v = T("fa_q").cuda(), T("fa_k").cuda(), T("fa_v").cuda()
    # fp16 operands on the matrix cores: P is rounded to fp16 before P V (the reference's own fp16 path does the
    # same, test/python/mlir/hexkl_attention/input.mlir:140-145), tolerance as in the parity tests
    got = hexmi.flash_attention(q, k, v, 1 / 8, False, out_dtype=torch.float32).cpu()
    assert (got - T("fa_o")).abs().max() <= 5e-3
    got = hexmi.flash_attention(q, k, v, 1 / 8, True, out_dtype=torch.float32).cpu()
    assert (got - T("fa_o_causal")).abs().max() <= 5e-3
    got = hexmi.attention(T("ma_q").cuda(), T("ma_k").cuda(), T("ma_v").cuda(), T("ma_mask").cuda(),
                          out_dtype=torch.float32).cpu()
    assert (got - T("ma_o")).abs().max() <= 5e-3


@pytest.mark.gpu
def test_hip_elementwise(hexmi):
    x = T("ew_x").cuda()
    assert close_half(hexmi.gelu(x).cpu(), T("gelu_y"), extra=2e-3 * 2.0 ** -10 + 1e-6)
    assert close_half(hexmi.silu(x).cpu(), T("silu_y"), extra=1e-6)
    assert close_half(hexmi.rope(T("rope_x").cuda(), 10000.0).cpu(), T("rope_y"), extra=1e-6)
    assert close32(hexmi.block_sum(T("sum_x").cuda(), 32).cpu(), T("sum_y"), 1e-6)
