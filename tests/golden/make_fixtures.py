"""Writes tests/golden/fixtures.npz: tiny seeded inputs and their expected outputs for every operator on the path.

The reference holds no numeric vectors of its own (its tests compare a device run with a PyTorch CPU call at run
time), so the expectations here come from the same PyTorch CPU library calls and closed forms the reference's
tests use as their oracle, evaluated in float64 on the stored (already rounded) inputs. Nothing from the
reference is imported or run. Re-run with `python tests/golden/make_fixtures.py`; the output is deterministic.
"""
import math
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    g = torch.Generator().manual_seed(20240607)
    out = {}

    def put(name, t):
        t = t.detach().cpu()
        out[name] = (t.float() if t.dtype == torch.float64 else t).numpy()     # expectations stored as fp32

    # row softmax, fp32 (test/python/triton/test_softmax.py:93: torch.softmax on the host)
    x = torch.randn(6, 37, generator=g)
    put("softmax_x", x)
    put("softmax_y", torch.softmax(x.double(), dim=-1))

    # RMSNorm / LayerNorm, fp16 in (test_rms_norm.py:85, test_layer_norm.py:111), eps 1e-5
    x = torch.randn(5, 48, generator=g).half()
    w = (1 + 0.1 * torch.randn(48, generator=g)).half()
    b = (0.1 * torch.randn(48, generator=g)).half()
    xd, wd, bd = x.double(), w.double(), b.double()
    put("norm_x", x), put("norm_w", w), put("norm_b", b)
    put("rms_y", xd * torch.rsqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * wd)
    mean = xd.mean(-1, keepdim=True)
    var = ((xd - mean) ** 2).mean(-1, keepdim=True)            # biased, two-pass (test_layer_norm.py:70)
    put("ln_y", (xd - mean) * torch.rsqrt(var + 1e-5) * wd + bd)
    put("ln_mean", mean.squeeze(-1)), put("ln_rstd", torch.rsqrt(var + 1e-5).squeeze(-1))

    # GEMM fp16 (test_matmul.py:90 torch.matmul), both operand orders
    a = (2 * torch.rand(24, 16, generator=g) - 1).half()
    bm = (2 * torch.rand(16, 40, generator=g) - 1).half()
    put("mm_a", a), put("mm_b", bm), put("mm_c", a.double() @ bm.double())

    # W8A16: C[m,n] = sum_k A[m,k] * (W[n,k] * s[n])
    a8 = torch.randn(3, 64, generator=g).half()
    w8 = torch.randint(-127, 128, (20, 64), generator=g, dtype=torch.int8)
    s8 = (0.001 + 0.019 * torch.rand(20, generator=g)).half()
    put("w8_a", a8), put("w8_w", w8), put("w8_s", s8)
    put("w8_c", (a8.double() @ w8.double().t()) * s8.double()[None, :])

    # attention [Z,H,S,D] fp16, scale 1/sqrt(D) (test_flash_attention.py:212 F.scaled_dot_product_attention)
    q, k, v = (torch.randn(1, 1, 40, 64, generator=g).half() for _ in range(3))
    put("fa_q", q), put("fa_k", k), put("fa_v", v)
    put("fa_o", F.scaled_dot_product_attention(q.double(), k.double(), v.double(), scale=1 / 8))
    put("fa_o_causal", F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=True, scale=1 / 8))

    # additive-mask attention [B,S,D] (LowerTmTensor.cpp:157-160)
    q3 = torch.randn(2, 16, 64, generator=g).half()
    k3, v3 = (torch.randn(2, 24, 64, generator=g).half() for _ in range(2))
    m3 = torch.randn(2, 16, 24, generator=g).half()
    put("ma_q", q3), put("ma_k", k3), put("ma_v", v3), put("ma_mask", m3)
    put("ma_o", F.scaled_dot_product_attention(q3.double(), k3.double(), v3.double(), attn_mask=m3.double()))

    # element-wise tutorials
    xe = (3 * torch.randn(64, generator=g)).half()
    put("ew_x", xe)
    put("gelu_y", F.gelu(xe.double(), approximate="tanh")), put("silu_y", F.silu(xe.double()))

    # RoPE over adjacent feature pairs: pair i of position m turns by m * theta^(-2i/F)
    xr = torch.randn(1, 5, 2, 8, generator=g).half()
    B, L, H, Fd = xr.shape
    xd = xr.double()
    pos = torch.arange(L, dtype=torch.float64)[:, None]
    inv = 10000.0 ** (-torch.arange(0, Fd, 2, dtype=torch.float64) / Fd)[None, :]
    ang = pos * inv                                              # [L, F/2]
    c, s = torch.cos(ang)[None, :, None, :], torch.sin(ang)[None, :, None, :]
    x0, x1 = xd[..., 0::2], xd[..., 1::2]
    yr = torch.empty_like(xd)
    yr[..., 0::2] = x0 * c - x1 * s
    yr[..., 1::2] = x0 * s + x1 * c
    put("rope_x", xr), put("rope_y", yr)

    # block sums, fp32 (test_sum.py:30-47)
    xs = torch.randn(4 * 32, generator=g)
    put("sum_x", xs), put("sum_y", xs.double().reshape(4, 32).sum(-1))

    np.savez_compressed(os.path.join(HERE, "fixtures.npz"), **out)
    print("wrote", os.path.join(HERE, "fixtures.npz"), "with", len(out), "arrays")


if __name__ == "__main__":
    main()
