"""Seeded synthetic inputs for the measured configurations.

All tensors are generated on the CPU with `torch.Generator().manual_seed(seed)`
so that a host oracle and the GPU kernels see identical bits; callers move
them to the device. Shapes, distributions and dtypes are the benchmark
configurations' (softmax fp32 [4096,1024]; norms fp16 [8192,4096]; GEMM fp16
4096^3 / bf16 8192^3; W8A16 M in {1,16,256}, N=11008, K=4096; causal attention
fp16 [4,32,4096,128] and [1,32,16384,128]).
"""
import math

import torch


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def softmax_inputs(rows=4096, cols=1024, dtype=torch.float32, seed=0):
    g = _gen(seed)
    return {"x": torch.randn(rows, cols, generator=g, dtype=torch.float32).to(dtype)}


def norm_inputs(rows=8192, cols=4096, dtype=torch.float16, seed=0):
    g = _gen(seed)
    x = torch.randn(rows, cols, generator=g, dtype=torch.float32).to(dtype)
    w = (1.0 + 0.1 * torch.randn(cols, generator=g, dtype=torch.float32)).to(dtype)
    b = (0.1 * torch.randn(cols, generator=g, dtype=torch.float32)).to(dtype)
    return {"x": x, "weight": w, "bias": b, "eps": 1e-5}


def gemm_inputs(M=4096, N=4096, K=4096, dtype=torch.float16, seed=0, trans_b=False):
    g = _gen(seed)
    a = (2.0 * torch.rand(M, K, generator=g, dtype=torch.float32) - 1.0).to(dtype)
    bshape = (N, K) if trans_b else (K, N)
    b = (2.0 * torch.rand(*bshape, generator=g, dtype=torch.float32) - 1.0).to(dtype)
    return {"a": a, "b": b}


def w8a16_inputs(M=16, N=11008, K=4096, seed=0):
    g = _gen(seed)
    a = torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.float16)
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    s = (0.001 + 0.019 * torch.rand(N, generator=g, dtype=torch.float32)).to(torch.float16)
    return {"a": a, "w": w, "scales": s}


def attention_inputs(Z=4, H=32, S=4096, D=128, dtype=torch.float16, seed=0):
    g = _gen(seed)
    q = torch.randn(Z, H, S, D, generator=g, dtype=torch.float32).to(dtype)
    k = torch.randn(Z, H, S, D, generator=g, dtype=torch.float32).to(dtype)
    v = torch.randn(Z, H, S, D, generator=g, dtype=torch.float32).to(dtype)
    return {"q": q, "k": k, "v": v, "sm_scale": 1.0 / math.sqrt(D)}


# Algorithmic work per launch: the bytes a perfect kernel must move (every
# input read once, every output written once) or the multiply-adds it must do.
def softmax_bytes(rows, cols, itemsize=4):
    return 2 * rows * cols * itemsize


def rms_norm_bytes(rows, cols, itemsize=2):
    return 2 * rows * cols * itemsize + cols * itemsize


def layer_norm_bytes(rows, cols, itemsize=2, stats=False):
    return 2 * rows * cols * itemsize + 2 * cols * itemsize + (8 * rows if stats else 0)


def gemm_flops(M, N, K):
    return 2 * M * N * K


def w8a16_bytes(M, N, K):
    return N * K + 2 * N + 2 * M * K + 2 * M * N


def attention_flops(Z, H, S, D, causal):
    full = 4 * Z * H * S * S * D
    return full // 2 if causal else full
