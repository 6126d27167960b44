#!/usr/bin/env python3
"""Roofline bench of the hexmi kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-suite] [--no-cpu]

Prints ONE JSON line. The headline `value` is the primary workload's throughput (default `norms`: one step =
RMSNorm + LayerNorm over the fp16 [8192, 4096] batch, GB/s of algorithmic bytes) with inputs resident in HBM
and the buffers rotated over > 512 MB so the 256 MB Infinity Cache cannot serve them. `suite` carries the same
measurement for every other configuration (GEMM / attention in TFLOP/s, W8A16 and softmax in GB/s), each with
its own roofline fraction. `cpu_baseline` times the reference's CPU path (the PyTorch CPU op its tests use as
oracle) on the host cores for the primary workload; suite entries carry their own `cpu` leg.

Kernel launch durations are measured with HIP events on the stream the kernels are launched on (torch's
current stream, which hexmi passes to the C ABI): the K steps are captured into one HIP graph and the graph is
replayed REPLAYS times, each replay timed on its own; `ms_per_step` is the median replay, `ms_min` the fastest.
`targets` lists the ten configurations that carry a throughput target with fraction, target and met / missed.
HBM-bound entries also carry a `hot` figure (one buffer set, served by the 256 MB Infinity Cache where it fits):
the rotated one is the HBM claim. `--workload mfma_peak` times a registers-only MFMA stream (zeros and U(-1,1)
operands, both instruction shapes, about a second each): the data-dependent ceiling of the matrix cores on this box.
`--workload issue_slots` (vector instructions that fit between a wave's MFMAs) and `--workload lds_patterns` (cycles
per LDS read for the GEMM's fragment address patterns) are two more calibrations of the same kind. `--operands zeros` runs a GEMM or attention workload on all-zero inputs
(same instructions, same traffic): against the random-operand time it shows what the data costs in power.
`--workload vendor` times the GEMM and attention configurations through this library and through torch.matmul /
F.scaled_dot_product_attention on the same box (a comparison; hexmi calls neither).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "hexagon-mlir_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0      # MI355X dense fp16 / bf16 matrix, published
MFMA_F32_PEAK_TFLOPS = 157.3   # MI355X fp32 matrix, published
ROTATE_BYTES = 1024 << 20      # rotate HBM-bound workloads over 4x the 256 MB Infinity Cache
REPLAYS = 7                    # timed replays of the K-step graph: median and min are reported
TARGETS = {                    # fraction of the published peak each configuration is asked to reach
    "softmax_f32_4096x1024": 0.70, "rms_norm_f16_8192x4096": 0.70, "layer_norm_f16_8192x4096": 0.70,
    "gemm_f16_4096": 0.60, "gemm_bf16_8192": 0.60, "w8a16_m1": 0.60, "w8a16_m16": 0.60, "w8a16_m256": 0.60,
    "attn_causal_f16_4x32x4096x128": 0.60, "attn_causal_f16_1x32x16384x128": 0.60,
}


class Workload:
    """One measured configuration: device buffers (several rotated sets), the launch, its algorithmic work."""

    name = ""
    bound = "hbm"
    dtype = ""
    work = 0                   # algorithmic bytes (hbm) or FLOP (mfma) per step
    desc = ""
    kernel = ""                # name of the dominant kernel as rocprofv3 reports it

    def setup(self, torch, hexmi):
        raise NotImplementedError

    def step(self, i):
        raise NotImplementedError

    def cpu(self, torch):
        """Returns (seconds per step-equivalent, sample description) for the reference's CPU path."""
        raise NotImplementedError


def _sets(torch, tensors, bytes_per_set, rotate=True):
    n = max(1, -(-ROTATE_BYTES // bytes_per_set)) if rotate else 1
    out = []
    for _ in range(min(n, 64)):                          # 64 sets of a small problem are out of every cache already
        out.append({k: (v.cuda() if hasattr(v, "cuda") else v) for k, v in tensors.items()})
    return out


class CopyCalibration(Workload):
    """Plain device copy of a known size (64 MiB read + 64 MiB written per step): the reference reading for scaling
    the FETCH_SIZE / WRITE_SIZE hardware counters to bytes. Not part of the suite."""
    name, bound, dtype, kernel = "copy_64MiB", "hbm", "u8", "elementwise copy (torch)"
    desc = "torch Tensor.copy_ of 64 MiB, 5 rotated sets"

    def setup(self, torch, hexmi):
        n = 64 << 20
        self.work = 2 * n
        self.sets = [{"x": torch.zeros(n, dtype=torch.uint8, device="cuda"),
                      "out": torch.empty(n, dtype=torch.uint8, device="cuda")} for _ in range(5)]

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        s["out"].copy_(s["x"])

    def cpu(self, torch):
        a = torch.zeros(64 << 20, dtype=torch.uint8)
        b = torch.empty_like(a)
        return _time_cpu(lambda: b.copy_(a), 3), "64 MiB memcpy on CPU"


class Softmax(Workload):
    bound, kernel = "hbm", "row_kernel"

    def __init__(self, rows=4096, cols=1024, dtype="f32"):
        self.rows, self.cols, self.dtype = rows, cols, dtype
        self.name = "softmax_%s_%dx%d" % (dtype, rows, cols)
        self.desc = "row softmax %s [%d,%d] N(0,1) seed 0" % (dtype, rows, cols)
        # few long rows: every row is cut into column blocks, two launches (statistics, then the normalising sweep)
        if rows < 128 and cols >= 16384:
            self.kernel = "part_stats_kernel + part_apply_kernel"

    def setup(self, torch, hexmi):
        from hexmi.workloads import softmax_inputs, softmax_bytes
        self.hexmi, self.host = hexmi, softmax_inputs(self.rows, self.cols)
        if self.dtype == "f16":
            self.host = {"x": self.host["x"].half()}
        self.work = softmax_bytes(self.rows, self.cols, 4 if self.dtype == "f32" else 2)
        self.sets = _sets(torch, self.host, self.work)
        for s in self.sets:
            s["out"] = torch.empty_like(s["x"])

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        self.hexmi.softmax(s["x"], out=s["out"])

    def cpu(self, torch):
        from oracle import torch_cpu
        x = self.host["x"][:4096].float()
        t = _time_cpu(lambda: torch_cpu.softmax(x), 5) * (self.rows / min(self.rows, 4096))
        return t, "rows 0..%d of [%d,%d], torch.softmax on CPU%s" % (min(self.rows, 4096), self.rows, self.cols,
                                                                    ", time scaled" if self.rows > 4096 else "")


class Norms(Workload):
    name, bound, dtype, kernel = "norms_f16_8192x4096", "hbm", "f16", "row_kernel"
    desc = "RMSNorm + LayerNorm fp16 [8192,4096] N(0,1), w~N(1,0.1), b~N(0,0.1), eps 1e-5, fp32 accumulation"
    which = ("rms", "ln")

    def setup(self, torch, hexmi):
        from hexmi.workloads import norm_inputs, rms_norm_bytes, layer_norm_bytes
        self.hexmi, self.host = hexmi, norm_inputs()
        self.work_rms, self.work_ln = rms_norm_bytes(8192, 4096), layer_norm_bytes(8192, 4096)
        self.work = (self.work_rms if "rms" in self.which else 0) + (self.work_ln if "ln" in self.which else 0)
        t = {k: v for k, v in self.host.items() if k != "eps"}
        self.sets = _sets(torch, t, self.work_rms)
        for s in self.sets:
            s["out"] = torch.empty_like(s["x"])

    def step(self, i):
        n = len(self.sets)
        s = self.sets[i % n]
        if "rms" in self.which:
            self.hexmi.rms_norm(s["x"], s["weight"], 1e-5, out=s["out"])
        if "ln" in self.which:
            # with both kernels in a step the second reads a set half the rotation away, not the 64 MiB the first
            # has just pulled through the Infinity Cache
            t = self.sets[(i + n // 2) % n] if "rms" in self.which else s
            self.hexmi.layer_norm(t["x"], t["weight"], t["bias"], 1e-5, out=t["out"])

    def cpu(self, torch):
        from oracle import torch_cpu
        h = self.host

        def run():
            if "rms" in self.which:
                torch_cpu.rms_norm(h["x"], h["weight"], 1e-5)
            if "ln" in self.which:
                torch_cpu.layer_norm(h["x"], h["weight"], h["bias"], 1e-5)
        return _time_cpu(run, 3), "full [8192,4096], F.rms_norm / F.layer_norm on CPU"


class RmsNorm(Norms):
    name, which = "rms_norm_f16_8192x4096", ("rms",)
    desc = "RMSNorm fp16 [8192,4096]"


class LayerNorm(Norms):
    name, which = "layer_norm_f16_8192x4096", ("ln",)
    desc = "LayerNorm fp16 [8192,4096]"


# --operands zeros: the matrix-core workloads (GEMM, attention) run on all-zero inputs, through the same
# instructions and the same memory traffic. Not a throughput claim: the difference to the random-operand time is what
# the data costs in power, and the line says so in its "data" field.
ZERO_OPERANDS = False


def _zero_operands(buffers, names):
    if ZERO_OPERANDS:
        for n in names:
            buffers[n].zero_()


class Gemm(Workload):
    bound, kernel = "mfma", "gemm_kernel_k64"

    def __init__(self, size, dtype_name, packed=False):
        self.size, self.dtype, self.packed = size, dtype_name, packed
        self.name = "gemm_%s_%d%s" % (dtype_name, size, "_packed_weight" if packed else "")
        self.desc = "C=A.B %s [%d,%d]x[%d,%d] U(-1,1), fp32 accumulate, %s out" % (dtype_name, size, size, size, size,
                                                                                   dtype_name)
        if packed:
            self.desc += "; B re-laid-out once to [N,K] (hexmi_transpose16, outside the timed region) and multiplied as B^T"

    def setup(self, torch, hexmi):
        from hexmi.workloads import gemm_inputs, gemm_flops
        dt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[self.dtype]
        if self.dtype == "f32":
            self.kernel, self.peak = "gemm_f32_mfma_kernel", MFMA_F32_PEAK_TFLOPS
        self.hexmi, self.host = hexmi, gemm_inputs(self.size, self.size, self.size, dt)
        self.work = gemm_flops(self.size, self.size, self.size)
        self.sets = _sets(torch, self.host, 0, rotate=False)
        self.sets[0]["out"] = torch.empty(self.size, self.size, dtype=dt, device="cuda")
        _zero_operands(self.sets[0], ("a", "b"))
        if self.packed:
            self.sets[0]["b"] = hexmi.pack_weight(self.sets[0]["b"])

    def step(self, i):
        s = self.sets[0]
        self.hexmi.matmul(s["a"], s["b"], out=s["out"], trans_b=self.packed)

    def cpu(self, torch):
        from oracle import torch_cpu
        n = self.size
        rows = n if n <= 4096 else n // 8
        a = self.host["a"][:rows]
        t = _time_cpu(lambda: torch_cpu.matmul(a, self.host["b"]), 1 if n > 4096 else 2)
        return t * (n / rows), "rows 0..%d of A (of %d) x full B, fp32 torch.matmul on CPU, time scaled to the full GEMM" % (rows, n)


class GemmNT(Workload):
    """A[M,K] x W[N,K]^T fp16 off the square benchmark shapes: a decode step (one row or sixteen: a stream of the
    weights, priced against HBM) and a vocabulary projection with an odd N (priced against the matrix cores)."""
    dtype = "f16"

    def __init__(self, M, N, K):
        self.M, self.N, self.K = M, N, K
        self.name = "gemm_f16_nt_%dx%dx%d" % (M, N, K)
        self.bound = "hbm" if M <= 64 else "mfma"
        self.kernel = "gemv_nt_kernel" if M <= 8 else ("gemm_nt_skinny_kernel" if M <= 64 else "gemm_kernel_k64")
        self.desc = "C = A[%d,%d] . W[%d,%d]^T fp16 U(-1,1), fp32 accumulate, fp16 out" % (M, K, N, K)

    def setup(self, torch, hexmi):
        from hexmi.workloads import gemm_inputs, gemm_flops
        self.hexmi, self.host = hexmi, gemm_inputs(self.M, self.N, self.K, torch.float16, trans_b=True)
        bytes_ = 2 * (self.N * self.K + self.M * self.K + self.M * self.N)
        self.work = bytes_ if self.bound == "hbm" else gemm_flops(self.M, self.N, self.K)
        self.sets = _sets(torch, self.host, bytes_, rotate=self.bound == "hbm")
        for s in self.sets:
            s["out"] = torch.empty(self.M, self.N, dtype=torch.float16, device="cuda")

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        self.hexmi.matmul(s["a"], s["b"], out=s["out"], trans_b=True)

    def cpu(self, torch):
        a, b = self.host["a"].float(), self.host["b"].float()
        rows = min(self.M, 512)
        t = _time_cpu(lambda: torch.matmul(a[:rows], b.t()), 2)
        return t * (self.M / rows), "rows 0..%d of %d, fp32 torch.matmul on CPU%s" % (rows, self.M, ", time scaled" if rows < self.M else "")


class W8A16(Workload):
    bound, dtype = "hbm", "f16"
    # the kernel rocprofv3 names for each measured shape (the library picks by M, N, K)
    KERNELS = {(1, 11008): "w8a16_gemv_kernel", (16, 11008): "w8a16_mid_kernel", (64, 11008): "w8a16_mid_kernel",
               (256, 11008): "gemm_kernel_k64", (1, 4096): "w8a16_gemv_any_kernel", (16, 4096): "w8a16_mid_kernel",
               (64, 4096): "w8a16_split_kernel", (256, 4096): "w8a16_split_kernel"}

    def __init__(self, M, N=11008, K=4096):
        self.M, self.N, self.K = M, N, K
        # N = 11008, K = 4096 is the measured configuration (a gate / up projection); N = 4096, K = 11008 is the down
        # projection of the same model: the same 45 MB of weights walked the other way
        self.name = ("w8a16_m%d" if N == 11008 else "w8a16_down_m%d") % M
        self.kernel = self.KERNELS.get((M, N), "w8a16")
        self.desc = ("W8A16 A fp16 [%d,%d] N(0,1), W int8 [%d,%d], per-channel fp16 scales, fp32 accumulate"
                     % (M, K, N, K))

    def setup(self, torch, hexmi):
        from hexmi.workloads import w8a16_inputs, w8a16_bytes
        self.hexmi, self.host = hexmi, w8a16_inputs(self.M, self.N, self.K)
        self.work = w8a16_bytes(self.M, self.N, self.K)
        self.sets = _sets(torch, self.host, self.work)
        for s in self.sets:
            s["out"] = torch.empty(self.M, self.N, dtype=torch.float16, device="cuda")

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        self.hexmi.w8a16_matmul(s["a"], s["w"], s["scales"], out=s["out"])

    def cpu(self, torch):
        from oracle import torch_cpu
        h = self.host
        return (_time_cpu(lambda: torch_cpu.w8a16_matmul(h["a"], h["w"], h["scales"]), 2),
                "full size, dequantise + fp32 matmul on CPU")


class W8A16Packed(W8A16):
    """The same product on weights pre-packed once into fragment-major order (not part of the timed step)."""

    def __init__(self, M):
        super().__init__(M)
        self.name = "w8a16_packed_m%d" % M
        self.kernel = "w8a16_persist_kernel"
        self.desc += ", weights pre-packed by hexmi_pack_w8"

    def setup(self, torch, hexmi):
        super().setup(torch, hexmi)
        for s in self.sets:
            s["wp"] = hexmi.pack_w8(s["w"])
            del s["w"]

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        self.hexmi.w8a16_matmul_packed(s["a"], s["wp"], s["scales"], out=s["out"])


class Attention(Workload):
    bound, dtype, kernel = "mfma", "f16", "flash_fwd_kernel"

    def __init__(self, Z, H, S, D):
        self.shape = (Z, H, S, D)
        self.name = "attn_causal_f16_%dx%dx%dx%d" % self.shape
        self.desc = "causal flash-attention fwd fp16 [%d,%d,%d,%d] N(0,1), scale 1/sqrt(%d), fp32 stats" % (Z, H, S, D, D)

    def setup(self, torch, hexmi):
        from hexmi.workloads import attention_inputs, attention_flops
        self.hexmi, self.host = hexmi, attention_inputs(*self.shape)
        self.work = attention_flops(*self.shape, causal=True)
        t = {k: v for k, v in self.host.items() if k != "sm_scale"}
        self.sets = _sets(torch, t, 0, rotate=False)
        self.sets[0]["out"] = torch.empty_like(self.sets[0]["q"])
        _zero_operands(self.sets[0], ("q", "k", "v"))

    def step(self, i):
        s = self.sets[0]
        self.hexmi.flash_attention(s["q"], s["k"], s["v"], self.host["sm_scale"], True, out=s["out"])

    def cpu(self, torch):
        from oracle import torch_cpu
        Z, H, S, D = self.shape
        heads = 8 if S <= 4096 else 2
        h = self.host
        q, k, v = (h[n].reshape(Z * H, S, D)[:heads][None] for n in ("q", "k", "v"))
        t = _time_cpu(lambda: torch_cpu.attention(q, k, v, h["sm_scale"], True), 1)
        return t * (Z * H / heads), "%d of %d heads, fp32 F.scaled_dot_product_attention(is_causal=True) on CPU, time scaled" % (heads, Z * H)


class AttentionF32(Attention):
    """The reference test's own dtype (fp32 Q, K, V: test/python/triton/test_flash_attention.py:171-173) at a size
    that fills the chip; priced against the fp32 matrix peak."""
    dtype, kernel, peak = "f32", "flash_fwd_f32_kernel", MFMA_F32_PEAK_TFLOPS

    def __init__(self, Z, H, S, D):
        self.shape = (Z, H, S, D)
        self.name = "attn_causal_f32_%dx%dx%dx%d" % self.shape
        self.desc = "causal flash-attention fwd fp32 [%d,%d,%d,%d] N(0,1), scale 1/sqrt(%d)" % (Z, H, S, D, D)

    def setup(self, torch, hexmi):
        from hexmi.workloads import attention_inputs, attention_flops
        self.hexmi, self.host = hexmi, attention_inputs(*self.shape, dtype=torch.float32)
        self.work = attention_flops(*self.shape, causal=True)
        t = {k: v for k, v in self.host.items() if k != "sm_scale"}
        self.sets = _sets(torch, t, 0, rotate=False)
        self.sets[0]["out"] = torch.empty_like(self.sets[0]["q"])


class Elementwise(Workload):
    """The reference's small tutorial kernels at a size that needs HBM: GELU-tanh / SiLU over fp16 [8192,4096],
    RoPE over fp16 [4,4096,32,128], one sum per 4096-element program over fp32 [8192*4096]."""
    bound = "hbm"

    def __init__(self, which):
        self.which = which
        self.name = {"gelu": "gelu_f16_8192x4096", "silu": "silu_f16_8192x4096", "rope": "rope_f16_4x4096x32x128",
                     "sum": "block_sum_f32_8192x4096"}[which]
        self.kernel = {"gelu": "unary_kernel", "silu": "unary_kernel", "rope": "rope_kernel", "sum": "block_sum_kernel"}[which]
        self.dtype = "f32" if which == "sum" else "f16"
        self.desc = {"gelu": "GELU-tanh fp16 [8192,4096] N(0,1)", "silu": "SiLU fp16 [8192,4096] N(0,1)",
                     "rope": "RoPE fp16 [batch 4, seq 4096, heads 32, features 128] N(0,1), theta 1e4",
                     "sum": "8192 programs x 4096 fp32 elements, one sum each"}[which]

    def setup(self, torch, hexmi):
        g = torch.Generator().manual_seed(0)
        self.hexmi = hexmi
        if self.which == "rope":
            x = torch.randn(4, 4096, 32, 128, generator=g).half()
        elif self.which == "sum":
            x = torch.randn(8192 * 4096, generator=g)
        else:
            x = torch.randn(8192, 4096, generator=g).half()
        self.host = {"x": x}
        n_bytes = x.numel() * x.element_size()
        self.work = n_bytes + 8192 * 4 if self.which == "sum" else 2 * n_bytes
        self.sets = _sets(torch, self.host, self.work)
        for s in self.sets:
            s["out"] = torch.empty(8192, device="cuda") if self.which == "sum" else torch.empty_like(s["x"])

    def step(self, i):
        s = self.sets[i % len(self.sets)]
        if self.which == "gelu":
            self.hexmi.gelu(s["x"], out=s["out"])
        elif self.which == "silu":
            self.hexmi.silu(s["x"], out=s["out"])
        elif self.which == "rope":
            self.hexmi.rope(s["x"], 10000.0, out=s["out"])
        else:
            self.hexmi.block_sum(s["x"], 4096, out=s["out"])

    def cpu(self, torch):
        import torch.nn.functional as F
        x = self.host["x"]
        if self.which == "gelu":
            return _time_cpu(lambda: F.gelu(x, approximate="tanh"), 3), "full tensor, F.gelu(approximate='tanh') on CPU"
        if self.which == "silu":
            return _time_cpu(lambda: F.silu(x), 3), "full tensor, F.silu on CPU"
        if self.which == "sum":
            return _time_cpu(lambda: x.view(8192, 4096).sum(1), 3), "full tensor, torch.sum(dim=1) on CPU"
        D, L = 128, 4096
        idx = torch.arange(D, dtype=torch.float32)
        steps = torch.where(idx % 2 == 0, idx, idx - 1)
        ang = torch.arange(L, dtype=torch.float32)[:, None] * (1.0 / (10000.0 ** (steps / D)))[None, :]
        cos, sin = torch.cos(ang).reshape(1, L, 1, D), torch.sin(ang).reshape(1, L, 1, D)
        even = (torch.arange(D) % 2 == 0).view(1, 1, 1, D)
        xs = x[:1]

        def run():
            torch.where(even, xs * cos - torch.roll(xs, -1, 3) * sin, torch.roll(xs, 1, 3) * sin + xs * cos)
        return _time_cpu(run, 1) * 4, "1 of 4 batch entries, the reference's torch RoPE formula on CPU, time scaled"


class MaskedAttention(Workload):
    """tm_tensor.attention with an additive mask (the next row after the causal kernel): [B,S,D] operands."""
    bound, dtype, kernel = "mfma", "f16", "flash_fwd_kernel"

    def __init__(self, B, S, D):
        self.shape = (B, S, D)
        self.name = "attn_masked_f16_%dx%dx%d" % self.shape
        self.desc = ("tm_tensor.attention fp16 q,k,v [%d,%d,%d] N(0,1), additive mask [%d,%d,%d] N(0,1) with 30%% -inf, "
                     "scale 1/sqrt(%d)" % (B, S, D, B, S, S, D))

    def setup(self, torch, hexmi):
        B, S, D = self.shape
        g = torch.Generator().manual_seed(0)
        q, k, v = (torch.randn(B, S, D, generator=g).half() for _ in range(3))
        mask = torch.randn(B, S, S, generator=g)
        mask[torch.rand(B, S, S, generator=g) < 0.3] = float("-inf")
        mask[:, :, 0] = 0.0
        self.hexmi, self.host = hexmi, {"q": q, "k": k, "v": v, "mask": mask.half()}
        self.work = 4 * B * S * S * D                     # QK^T and PV, every key of every query
        self.sets = _sets(torch, self.host, 0, rotate=False)
        self.sets[0]["out"] = torch.empty_like(self.sets[0]["q"])

    def step(self, i):
        s = self.sets[0]
        self.hexmi.attention(s["q"], s["k"], s["v"], s["mask"], out=s["out"])

    def cpu(self, torch):
        from oracle import torch_cpu
        B, S, D = self.shape
        n = 4
        h = self.host
        t = _time_cpu(lambda: torch_cpu.attention_masked(h["q"][:n], h["k"][:n], h["v"][:n], h["mask"][:n],
                                                         1.0 / math.sqrt(D)), 1)
        return t * (B / n), "%d of %d batch entries, fp32 F.scaled_dot_product_attention(attn_mask=...) on CPU, time scaled" % (n, B)


class LinearFused(Workload):
    """A GPT-2 style projection with bias and residual: one launch (hexmi_gemm_ex) against the same result from the
    GEMM followed by two element-wise add launches."""
    bound, kernel, dtype = "mfma", "gemm_kernel_k64", "f16"
    launches_separate = 3

    def __init__(self, M=8192, N=768, K=3072):
        self.M, self.N, self.K = M, N, K
        self.name = "linear_bias_residual_f16_%dx%dx%d" % (M, N, K)
        self.desc = ("C = A[%d,%d].B[%d,%d] + bias[%d] + residual[%d,%d], fp16, fp32 accumulate, one rounding; "
                     "the GPT-2 small MLP projection over 8 sequences of 1024 tokens" % (M, K, K, N, N, M, N))

    def setup(self, torch, hexmi):
        g = torch.Generator().manual_seed(7)
        self.hexmi = hexmi
        self.host = {"a": torch.rand(self.M, self.K, generator=g).mul_(2).sub_(1).half(),
                     "b": torch.rand(self.K, self.N, generator=g).mul_(2).sub_(1).half(),
                     "bias": torch.rand(self.N, generator=g).half(),
                     "resid": torch.rand(self.M, self.N, generator=g).half()}
        self.work = 2.0 * self.M * self.N * self.K
        self.sets = _sets(torch, self.host, 0, rotate=False)
        s = self.sets[0]
        s["out"] = torch.empty(self.M, self.N, dtype=torch.float16, device="cuda")
        s["tmp"] = torch.empty_like(s["out"])
        s["bias_rows"] = s["bias"].expand(self.M, self.N).contiguous()

    def step(self, i):
        s = self.sets[0]
        self.hexmi.matmul(s["a"], s["b"], out=s["out"], bias=s["bias"], residual=s["resid"])

    def step_separate(self, i):
        s = self.sets[0]
        self.hexmi.matmul(s["a"], s["b"], out=s["tmp"])
        self.hexmi.binary("add", s["tmp"], s["bias_rows"], out=s["tmp"])
        self.hexmi.binary("add", s["tmp"], s["resid"], out=s["out"])

    def cpu(self, torch):
        a, b = self.host["a"].float(), self.host["b"].float()
        bias, resid = self.host["bias"].float(), self.host["resid"].float()
        rows = self.M // 8
        t = _time_cpu(lambda: torch.addmm(resid[:rows] + bias, a[:rows], b), 2)
        return t * 8, "rows 0..%d of %d, fp32 torch.addmm on CPU, time scaled to the full product" % (rows, self.M)


class AddMatmulSoftmax(Workload):
    """softmax((x + y) z) in one launch against add -> GEMM -> softmax (three launches)."""
    bound, kernel = "mfma", "add_matmul_softmax_kernel"
    launches_separate = 3

    def __init__(self, M, N, K, dtype_name):
        self.M, self.N, self.K, self.dtype = M, N, K, dtype_name
        self.name = "add_matmul_softmax_%s_%dx%dx%d" % (dtype_name, M, N, K)
        self.desc = "softmax((x + y)[%d,%d] . z[%d,%d]) over rows, %s, N(0,1) inputs" % (M, K, K, N, dtype_name)

    def setup(self, torch, hexmi):
        dt = {"f16": torch.float16, "f32": torch.float32}[self.dtype]
        if self.dtype == "f32":
            self.peak = MFMA_F32_PEAK_TFLOPS
        g = torch.Generator().manual_seed(9)
        self.hexmi = hexmi
        if self.M * self.N * self.K > hexmi.ops._FUSED_MAX_MACS:       # the operator then runs the three kernels
            self.kernel = "binary_kernel + gemm_kernel_k64 + row_kernel"
        self.host = {"x": torch.randn(self.M, self.K, generator=g).to(dt), "y": torch.randn(self.M, self.K, generator=g).to(dt),
                     "z": torch.randn(self.K, self.N, generator=g).mul_(self.K ** -0.5).to(dt)}
        self.work = 2.0 * self.M * self.N * self.K
        self.sets = _sets(torch, self.host, 0, rotate=False)
        self.sets[0]["out"] = torch.empty(self.M, self.N, dtype=dt, device="cuda")

    def step(self, i):
        # the path the operator takes by itself at this size (one launch for small products, three beyond)
        s = self.sets[0]
        self.hexmi.add_matmul_softmax(s["x"], s["y"], s["z"], out=s["out"])

    def step_fused(self, i):
        s = self.sets[0]
        self.hexmi.add_matmul_softmax(s["x"], s["y"], s["z"], out=s["out"], fused=True)

    def step_separate(self, i):
        s = self.sets[0]
        self.hexmi.add_matmul_softmax(s["x"], s["y"], s["z"], out=s["out"], fused=False)

    def cpu(self, torch):
        x, y, z = (self.host[k].float() for k in "xyz")
        t = _time_cpu(lambda: torch.softmax((x + y) @ z, dim=-1), 5)
        return t, "the whole graph, fp32 torch on CPU"


class MfmaPeak(Workload):
    """Registers-only MFMA stream (hexmi_mfma_peak): the rate the matrix cores sustain on given operand data."""
    bound, kernel = "mfma", "mfma_peak_kernel"

    def __init__(self, shape, dtype_name, data, waves=2):
        self.shape, self.dtype, self.data, self.waves = shape, dtype_name, data, waves
        tag = ("32x32x16", "16x16x32", "16x16x32_tile8x8")[shape]
        if shape == 2:
            self.waves = waves = 1
        self.name = "mfma_peak_%s_%s_%s" % (tag, dtype_name, data)
        self.desc = ("v_mfma_f32_%s_%s only, %d waves per SIMD, operands %s, accumulators in registers%s"
                     % (tag[:8], dtype_name, waves, "all zero" if data == "zeros" else "U(-1,1)",
                        ", 8 A x 8 B fragments walked as a GEMM tile (one operand changes per instruction)" if shape == 2 else ""))
        self.iters = 5000 if shape == 2 else 20000

    def setup(self, torch, hexmi):
        from hexmi import _lib
        self.lib, self._lib = _lib.lib(), _lib
        dt = torch.float16 if self.dtype == "f16" else torch.bfloat16
        g = torch.Generator().manual_seed(0)
        n_ops = 8192 if self.shape == 2 else 1024
        ops = torch.zeros(n_ops) if self.data == "zeros" else 2 * torch.rand(n_ops, generator=g) - 1
        self.ops = ops.to(dt).cuda()
        self.sink = torch.empty(self.lib.hexmi_num_cus() * 256 * self.waves, device="cuda")
        self.work = int(self.lib.hexmi_mfma_peak_flops(self.shape, self.waves, self.iters))
        self.code = _lib.F16 if self.dtype == "f16" else _lib.BF16
        self.stream = torch.cuda.current_stream
        self.sets = [None]

    def step(self, i):
        self._lib.check(self.lib.hexmi_mfma_peak(self.shape, self.code, self.ops.data_ptr(), self.iters, self.waves,
                                                 self.sink.data_ptr(), self.stream().cuda_stream), "hexmi_mfma_peak")

    def cpu(self, torch):
        return float("nan"), "no CPU counterpart"


def _time_cpu(fn, iters):
    fn()                                                # warm-up
    ts = []
    for _ in range(iters):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2]


def make_workloads():
    return {w.name: w for w in (
        Norms(), Softmax(), Softmax(65536, 1024), Softmax(4, 65536, "f16"), Softmax(16, 131072), RmsNorm(), LayerNorm(), Gemm(4096, "f16"), Gemm(8192, "bf16"),
        Gemm(8192, "bf16", packed=True), Gemm(4096, "f32"), W8A16(1), W8A16(16), W8A16Packed(16), W8A16(64), W8A16(256),
        W8A16(1, 4096, 11008), W8A16(16, 4096, 11008), W8A16(64, 4096, 11008), W8A16(256, 4096, 11008),
        Attention(4, 32, 4096, 128), Attention(1, 32, 16384, 128), AttentionF32(4, 32, 2048, 64),
        # off the kernels' own shapes: head sizes on padded tiles / two halves, ragged rows, [N,K] weights with one
        # row and with an odd N
        Attention(2, 16, 2048, 80), Attention(2, 16, 2048, 256), Softmax(8192, 50257, "f16"),
        GemmNT(1, 4096, 4096), GemmNT(16, 4096, 4096), GemmNT(4096, 50257, 768),
        MaskedAttention(32, 2048, 128), Elementwise("gelu"), Elementwise("silu"), Elementwise("rope"),
        Elementwise("sum"), LinearFused(), AddMatmulSoftmax(32, 32, 32, "f32"), AddMatmulSoftmax(512, 512, 64, "f16"),
        CopyCalibration())}


def peak_workloads():
    return ([MfmaPeak(shape, dt, data) for dt in ("f16", "bf16") for shape in (0, 1) for data in ("zeros", "uniform")]
            + [MfmaPeak(2, dt, "uniform") for dt in ("f16", "bf16")])


ALIASES = {"copy": "copy_64MiB", "norms": "norms_f16_8192x4096", "softmax": "softmax_f32_4096x1024",
           "softmax_big": "softmax_f32_65536x1024", "gemm": "gemm_f16_4096",
           "gemm_bf16": "gemm_bf16_8192", "gemm_bf16_packed": "gemm_bf16_8192_packed_weight", "gemm_f32": "gemm_f32_4096", "attn": "attn_causal_f16_4x32x4096x128",
           "attn_long": "attn_causal_f16_1x32x16384x128", "attn_masked": "attn_masked_f16_32x2048x128",
           "attn_f32": "attn_causal_f32_4x32x2048x64", "gelu": "gelu_f16_8192x4096", "silu": "silu_f16_8192x4096",
           "rope": "rope_f16_4x4096x32x128", "sum": "block_sum_f32_8192x4096", "rms_norm": "rms_norm_f16_8192x4096",
           "layer_norm": "layer_norm_f16_8192x4096", "w8a16_m1": "w8a16_m1", "w8a16_m16": "w8a16_m16",
           "w8a16_m64": "w8a16_m64", "w8a16_m256": "w8a16_m256", "w8a16_down_m1": "w8a16_down_m1",
           "w8a16_down_m16": "w8a16_down_m16", "w8a16_down_m64": "w8a16_down_m64", "w8a16_down_m256": "w8a16_down_m256",
           "linear": "linear_bias_residual_f16_8192x768x3072", "ams": "add_matmul_softmax_f32_32x32x32",
           "ams_mid": "add_matmul_softmax_f16_512x512x64"}


def measure(torch, wl, steps, warmup, use_graph=True, replays=REPLAYS):
    """Per-step times (ms) from HIP events on the current stream: {"ms": median, "min": ..., "max": ...,
    "wall": host wall-clock ms per step of the same replays, "graph": bool}.

    The K steps are captured once into a HIP graph; the graph is replayed `replays` times and every replay (exactly
    K steps) is timed on its own, so the figure is the GPU's time for back-to-back launches and not the host's launch
    cadence (a Python -> ctypes launch costs more than the shortest kernels here run). Falls back to direct launches
    if capture is unavailable."""
    for i in range(warmup):
        wl.step(i)
    torch.cuda.synchronize()
    graph = None
    if use_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(steps):
                    wl.step(warmup + i)
            graph.replay()                              # untimed: first replay pays the upload
            torch.cuda.synchronize()
        except Exception as exc:                        # noqa: BLE001 - report and fall back
            print("# graph capture failed (%s); timing direct launches" % exc, file=sys.stderr)
            graph = None
            torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(replays)]
    t0 = time.perf_counter()
    for e0, e1 in events:
        e0.record()
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                wl.step(warmup + i)
        e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / (steps * replays)
    per = sorted(e0.elapsed_time(e1) / steps for e0, e1 in events)
    return {"ms": per[len(per) // 2], "min": per[0], "max": per[-1], "wall": wall_ms, "graph": graph is not None,
            "replays": replays}


def measure_hot(torch, wl, steps, warmup, use_graph):
    """The same steps on ONE buffer set (what the Infinity Cache serves when the set fits in it), or None."""
    if wl.bound != "hbm" or not wl.sets or len(wl.sets) < 2:
        return None
    all_sets, wl.sets = wl.sets, wl.sets[:1]
    try:
        return measure(torch, wl, steps, warmup, use_graph, replays=3)
    finally:
        wl.sets = all_sets


def measured_traffic(wl):
    """HBM bytes per step from the committed rocprofv3 counter runs (profiles/traffic.json), or None."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            table = json.load(f)["traffic"]
        per_kernel = table[wl.name]
        return sum(per_kernel.values())
    except (OSError, KeyError, ValueError):
        return None


def report(wl, ms):
    if wl.bound == "hbm":
        achieved, peak, unit = wl.work / (ms * 1e-3) / 1e9, HBM_PEAK_GBS, "GB/s"
    else:
        achieved, peak, unit = wl.work / (ms * 1e-3) / 1e12, getattr(wl, "peak", MFMA_PEAK_TFLOPS), "TFLOP/s"
    return {"bound": wl.bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": measured_traffic(wl), "kernel": wl.kernel,
            "work_per_step": wl.work}


def box_calibration(torch, hexmi):
    """This box's own ceilings, measured in the same run as everything else (boxes of one pool differ by 10 % and
    more): what a plain device copy moves, and what the matrix cores sustain on U(-1,1) operands in a registers-only
    stream of the instruction the GEMM is built on. A fraction of the published peak can be read against these."""
    copy = CopyCalibration()
    copy.setup(torch, hexmi)
    cm = measure(torch, copy, 20, 3, use_graph=True, replays=3)
    copy_gbs = copy.work / (cm["ms"] * 1e-3) / 1e9
    copy.sets = None
    peak = MfmaPeak(1, "f16", "uniform")
    peak.iters = 4000                                   # about 40 ms per launch
    peak.setup(torch, hexmi)
    pm = measure(torch, peak, 3, 1, use_graph=False, replays=3)
    mfma_tf = peak.work / (pm["ms"] * 1e-3) / 1e12
    torch.cuda.empty_cache()
    return {"copy_64MiB_GBs": round(copy_gbs, 1), "copy_frac_of_hbm_peak": round(copy_gbs / HBM_PEAK_GBS, 4),
            "mfma_16x16x32_f16_uniform_TFLOPs": round(mfma_tf, 1),
            "mfma_frac_of_peak": round(mfma_tf / MFMA_PEAK_TFLOPS, 4),
            "note": "measured in this run on this box: a device copy (read + write bytes) and a registers-only MFMA "
                    "stream on U(-1,1) data; the fractions in this line stay against the published peaks"}


def steps_for(wl, steps):
    if wl.name.startswith("gemm_bf16_8192") or wl.name.startswith("gemm_f32") or "16384" in wl.name:
        return max(5, steps // 5)
    return steps


def entry_for(torch, wl, m, hot, cores, with_cpu):
    entry = {"workload": wl.name, "ms": round(m["ms"], 5), "ms_min": round(m["min"], 5), "ms_max": round(m["max"], 5),
             "replays": m["replays"]}
    entry.update(report(wl, m["ms"]))
    entry["frac_best"] = round(report(wl, m["min"])["frac"], 4)
    if hot is not None:
        entry["hot"] = {"ms": round(hot["ms"], 5), "frac": report(wl, hot["ms"])["frac"],
                        "note": "one buffer set: Infinity-Cache resident where it fits, not an HBM figure"}
    if wl.name in ("w8a16_m256", "w8a16_down_m256"):
        # 23 GFLOP: this shape is matrix-bound, not weight-stream-bound; both fractions are reported
        flop = 2.0 * 256 * 11008 * 4096
        entry["mfma_frac"] = round(flop / (m["ms"] * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)
    if with_cpu:
        sec, sample = wl.cpu(torch)
        if sec == sec:                                  # not NaN
            entry["cpu"] = {"ms": round(sec * 1e3, 3), "cores": cores, "sample": sample,
                            "value": round(wl.work / sec / (1e9 if wl.bound == "hbm" else 1e12), 4)}
    return entry


def direct_launch_cost(torch, wl, steps=300):
    """Host wall-clock per call (us) of direct launches from Python, GPU idle-waited only at the end."""
    for i in range(20):
        wl.step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        wl.step(i)
    host = (time.perf_counter() - t0) * 1e6 / steps     # time to enqueue
    torch.cuda.synchronize()
    total = (time.perf_counter() - t0) * 1e6 / steps    # enqueue + drain
    return {"host_us_per_call": round(host, 2), "wall_us_per_call": round(total, 2)}


def run_peak(torch, hexmi, args):
    """--workload mfma_peak: one JSON line with the sustained rate of every (dtype, shape, data) combination."""
    rows = []
    for wl in peak_workloads():
        wl.setup(torch, hexmi)
        wl.step(0)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        wl.step(0)
        e1.record()
        torch.cuda.synchronize()
        one = e0.elapsed_time(e1)
        k = max(5, int(math.ceil(1000.0 / max(one, 1e-3) / REPLAYS)))    # >= 1 s of back-to-back launches in all
        m = measure(torch, wl, k, 2, not args.no_graph)
        r = report(wl, m["ms"])
        rows.append({"workload": wl.name, "description": wl.desc, "ms": round(m["ms"], 4), "ms_min": round(m["min"], 4),
                     "launches": k * m["replays"], "sustained_s": round(m["ms"] * k * m["replays"] / 1e3, 2),
                     "achieved": r["achieved"], "unit": r["unit"], "frac": r["frac"],
                     "frac_best": report(wl, m["min"])["frac"],
                     "equivalent_clock_ghz": round(r["frac"] * 2.4, 3)})
        print("# %s: %.1f TFLOP/s (%.3f of peak)" % (wl.name, r["achieved"], r["frac"]), file=sys.stderr, flush=True)
    best = max(rows, key=lambda r: r["achieved"])
    line = {"metric": "GEMM/attn TFLOP/s + softmax/norm GB/s, % of MI355X roofline, 1 GPU", "value": best["achieved"],
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": best["ms"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16/bf16", "data": "synthetic",
            "config": {"workload": "mfma_peak", "description": "registers-only MFMA streams, a calibration of the "
                       "matrix cores' data-dependent ceiling, not a product kernel; equivalent_clock_ghz = fraction "
                       "of the published peak x the 2.4 GHz it is quoted at"},
            "roofline": {"bound": "mfma", "achieved": best["achieved"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": best["frac"], "traffic": None, "kernel": "mfma_peak_kernel"},
            "mfma_peak": rows}
    print(json.dumps(line), flush=True)


def _time_launch(torch, fn, repeats=5):
    """Median and minimum of `repeats` single launches (ms), HIP events on torch's current stream."""
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1))
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def _calibration_line(args, workload, description, kernel, rows, key):
    return {"metric": "GEMM/attn TFLOP/s + softmax/norm GB/s, % of MI355X roofline, 1 GPU", "value": None,
            "unit": "cycles", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None,
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": workload, "description": description},
            "roofline": {"bound": "mfma", "achieved": None, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": None,
                         "traffic": None, "kernel": kernel},
            key: rows}


def run_issue_slots(torch, hexmi, args):
    """--workload issue_slots: time per MFMA of a registers-only stream with 0..8 vector instructions after each
    MFMA (hexmi_issue_slots; zero operands, so the clock is the 2.4 GHz the cycle figures assume)."""
    from hexmi import _lib
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 512, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    kinds = ["v_pk_add_f16", "v_fma_f32", "v_exp_f32", "v_fma_mix_f32", "v_cvt_f32_f16"]
    rows = []
    for waves in (1, 2):
        for shape in (1, 0):
            per_iter = 4 if shape == 0 else 16
            iters = 40000 if shape == 0 else 10000
            for kind in (0, 2) if shape == 1 else (0, 1, 2, 3, 4):
                for per in (0, 1, 2, 3, 4, 5, 6, 8):
                    fn = lambda: _lib.check(lib.hexmi_issue_slots(shape, kind, per, iters, waves, sink.data_ptr(), st),
                                            "hexmi_issue_slots")
                    med, best = _time_launch(torch, fn)
                    ns = med * 1e6 / (iters * per_iter * waves)
                    rows.append({"mfma": "32x32x16" if shape == 0 else "16x16x32", "waves_per_simd": waves,
                                 "instruction": kinds[kind], "per_mfma": per, "ns_per_mfma": round(ns, 2),
                                 "cycles_per_mfma_at_2.4GHz": round(ns * 2.4, 1), "launch_ms": round(med, 3),
                                 "launch_ms_min": round(best, 3)})
                    print("# %s, %d waves/SIMD, %d x %s per MFMA: %.1f cycles per MFMA" % (
                        rows[-1]["mfma"], waves, per, kinds[kind], ns * 2.4), file=sys.stderr, flush=True)
    print(json.dumps(_calibration_line(args, "issue_slots", "vector instructions between the MFMAs of one wave: time "
                                       "per MFMA per SIMD; a calibration, not a product kernel", "issue_slots_kernel",
                                       rows, "issue_slots")), flush=True)


class _Lambda:
    """A step function with the attributes measure() looks at."""
    sets = None

    def __init__(self, fn):
        self.step = (lambda i: fn()) if fn is not None else None


def run_vendor(torch, hexmi, args):
    """--workload vendor: the GEMM and causal-attention configurations through this library and through the
    libraries PyTorch-ROCm ships (torch.matmul -> hipBLASLt / rocBLAS, F.scaled_dot_product_attention), same box, same
    buffers, same HIP-graph protocol, alternating. A comparison, not a product path: nothing in hexmi calls them."""
    import torch.nn.functional as F
    from hexmi.workloads import gemm_inputs, gemm_flops, attention_inputs, attention_flops
    rows = []

    def pair(name, flops, ours, theirs, their_name, steps):
        for who, fn in (("hexmi", ours), (their_name, theirs), ("hexmi", ours), (their_name, theirs)):
            m = measure(torch, _Lambda(fn), steps, args.warmup, not args.no_graph)
            rows.append({"config": name, "library": who, "ms": round(m["ms"], 5), "ms_min": round(m["min"], 5),
                         "tflops": round(flops / (m["ms"] * 1e-3) / 1e12, 1),
                         "frac": round(flops / (m["ms"] * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4)})
            print("# %-34s %-28s %.4f ms  frac %.3f" % (name, who, rows[-1]["ms"], rows[-1]["frac"]), file=sys.stderr)

    for size, dt, tag in ((4096, torch.float16, "f16"), (8192, torch.bfloat16, "bf16")):
        host = gemm_inputs(size, size, size, dt)
        a, b = host["a"].cuda(), host["b"].cuda()
        out = torch.empty(size, size, dtype=dt, device="cuda")
        steps = args.steps if size <= 4096 else max(5, args.steps // 5)
        pair("gemm_%s_%d" % (tag, size), gemm_flops(size, size, size), lambda: hexmi.matmul(a, b, out=out),
             lambda: torch.matmul(a, b, out=out), "torch.matmul", steps)
        del a, b, out
    for shape in ((4, 32, 4096, 128), (1, 32, 16384, 128)):
        host = attention_inputs(*shape)
        q, k, v = host["q"].cuda(), host["k"].cuda(), host["v"].cuda()
        out = torch.empty_like(q)
        scale = host["sm_scale"]
        steps = args.steps if shape[2] <= 4096 else max(5, args.steps // 5)
        pair("attn_causal_f16_%dx%dx%dx%d" % shape, attention_flops(*shape, causal=True),
             lambda: hexmi.flash_attention(q, k, v, scale, True, out=out),
             lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=scale),
             "F.scaled_dot_product_attention", steps)
        del q, k, v, out
    # the row kernels against torch's own, on buffer sets rotated over 1 GiB (the Infinity Cache cannot serve them)
    from hexmi.workloads import (softmax_inputs, norm_inputs, softmax_bytes, rms_norm_bytes, layer_norm_bytes)

    def pair_hbm(name, nbytes, ours, theirs, their_name, n_sets):
        for who, fn in (("hexmi", ours), (their_name, theirs), ("hexmi", ours), (their_name, theirs)):
            wl = _Lambda(None)
            wl.step = lambda i, fn=fn: fn(i % n_sets)
            m = measure(torch, wl, args.steps, args.warmup, not args.no_graph)
            rows.append({"config": name, "library": who, "ms": round(m["ms"], 5), "ms_min": round(m["min"], 5),
                         "gbs": round(nbytes / (m["ms"] * 1e-3) / 1e9, 1),
                         "frac": round(nbytes / (m["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
            print("# %-34s %-28s %.4f ms  frac %.3f" % (name, who, rows[-1]["ms"], rows[-1]["frac"]), file=sys.stderr)

    host = softmax_inputs()
    xs = [host["x"].cuda() for _ in range(32)]
    outs = [torch.empty_like(x) for x in xs]
    pair_hbm("softmax_f32_4096x1024", softmax_bytes(4096, 1024), lambda j: hexmi.softmax(xs[j], out=outs[j]),
             lambda j: torch.softmax(xs[j], dim=-1), "torch.softmax", 32)
    del xs, outs
    host = norm_inputs()
    xs = [host["x"].cuda() for _ in range(8)]
    outs = [torch.empty_like(x) for x in xs]
    w, b = host["weight"].cuda(), host["bias"].cuda()
    pair_hbm("rms_norm_f16_8192x4096", rms_norm_bytes(8192, 4096), lambda j: hexmi.rms_norm(xs[j], w, 1e-5, out=outs[j]),
             lambda j: F.rms_norm(xs[j], (4096,), w, 1e-5), "F.rms_norm", 8)
    pair_hbm("layer_norm_f16_8192x4096", layer_norm_bytes(8192, 4096),
             lambda j: hexmi.layer_norm(xs[j], w, b, 1e-5, out=outs[j]),
             lambda j: F.layer_norm(xs[j], (4096,), w, b, 1e-5), "F.layer_norm", 8)
    del xs, outs
    print(json.dumps(_calibration_line(args, "vendor", "hexmi and the libraries PyTorch-ROCm ships on the same "
                                       "configurations, same box, alternating; fractions of 2.5 PFLOP/s (of 8 TB/s for the row kernels)",
                                       "gemm_kernel_k64 / flash_fwd_kernel", rows, "vendor")))


def run_lds_patterns(torch, hexmi, args):
    """--workload lds_patterns: cycles per wave-wide 16-byte LDS read for the tiled GEMM's fragment-read address
    patterns, the LDS saturated by 16 waves per compute unit (hexmi_lds_read_pattern)."""
    from hexmi import _lib
    lib = _lib.lib()
    sink = torch.empty(lib.hexmi_num_cus() * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    names = ["linear (lane * 16)", "fp16 rows, chunk 4*step + g, swizzle (row>>1)&7 (fp16 kernels)",
             "fp16 rows, chunk 2*g + step, swizzle (row>>1)&7", "fp16 rows, chunk 2*g + step, swizzle of the int8-weight kernel",
             "int8 rows, swizzle (row>>2)&3", "int8 rows, swizzle (row>>1)&3 (in use)", "fp16 rows, chunk 4*step + g, no swizzle"]
    iters = 20000
    # clock: the same launch shape on the linear pattern moves 1 KiB per read; the figure is quoted in ns and in
    # cycles of the 2.4 GHz the chip holds on a load this light
    rows = []
    for pat, name in enumerate(names):
        fn = lambda: _lib.check(lib.hexmi_lds_read_pattern(pat, iters, sink.data_ptr(), st), "hexmi_lds_read_pattern")
        med, best = _time_launch(torch, fn)
        ns = med * 1e6 / (iters * 8 * 16)                # per wave-wide read of one compute unit
        rows.append({"pattern": pat, "description": name, "ns_per_read": round(ns, 3),
                     "cycles_per_read_at_2.4GHz": round(ns * 2.4, 2), "bytes_per_cycle_per_cu": round(1024 / (ns * 2.4), 1),
                     "launch_ms": round(med, 3), "launch_ms_min": round(best, 3)})
        print("# pattern %d (%s): %.2f cycles per read" % (pat, name, ns * 2.4), file=sys.stderr, flush=True)
    print(json.dumps(_calibration_line(args, "lds_patterns", "wave-wide 16-byte LDS reads with the tiled GEMM's "
                                       "fragment address patterns; a calibration, not a product kernel",
                                       "lds_pattern_kernel", rows, "lds_patterns")), flush=True)


def run_l2_stream(torch, hexmi, args):
    """--workload l2_stream: what the compute units take in from L2 (hexmi_l2_stream): one workgroup of 16 waves per
    CU streaming a cache-resident region into LDS or into registers, every CU the same region or each its own; the
    last case streams regions far larger than the caches, for the same loop's rate from HBM."""
    from hexmi import _lib
    lib = _lib.lib()
    cus = lib.hexmi_num_cus()
    sink = torch.empty(cus * 1024, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    rows = []
    for region_kib, shared in ((512, 1), (64, 1), (64, 0), (8192, 0)):     # the last: 2 GiB over the grid, from HBM
        region = region_kib << 10
        src = torch.randint(0, 255, (region * (1 if shared else cus),), dtype=torch.uint8, device="cuda")
        for to_lds in (1, 0):
            passes = max(1, (2 << 30) // (region * 8))     # 256 MiB through every CU per launch
            fn = lambda: _lib.check(lib.hexmi_l2_stream(to_lds, shared, region, passes, src.data_ptr(), sink.data_ptr(), st),
                                    "hexmi_l2_stream")
            med, best = _time_launch(torch, fn)
            moved = cus * passes * region
            rows.append({"region_KiB": region_kib, "every_cu_the_same_region": bool(shared), "into": "LDS" if to_lds else "registers",
                         "TBs": round(moved / (med * 1e-3) / 1e12, 2), "GBs_per_cu": round(moved / cus / (med * 1e-3) / 1e9, 1),
                         "launch_ms": round(med, 3), "launch_ms_min": round(best, 3)})
            print("# %d KiB, %s, into %s: %.1f GB/s per CU" % (region_kib, "shared" if shared else "own region",
                                                               rows[-1]["into"], rows[-1]["GBs_per_cu"]), file=sys.stderr, flush=True)
        del src
    print(json.dumps(_calibration_line(args, "l2_stream", "16 waves per CU streaming an L2-resident region in 1 KiB pieces; "
                                       "a calibration, not a product kernel", "l2_stream_kernel", rows, "l2_stream")), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="norms")
    ap.add_argument("--no-suite", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-box", action="store_true", help="skip the box calibration (copy and MFMA rates of this box)")
    ap.add_argument("--no-graph", action="store_true", help="time direct launches instead of a HIP graph replay")
    ap.add_argument("--only", default="", help="comma-separated suite entries to measure (default: all)")
    ap.add_argument("--operands", choices=("random", "zeros"), default="random",
                    help="zeros: GEMM / attention workloads on all-zero inputs (what the data costs in power)")
    args = ap.parse_args()
    global ZERO_OPERANDS
    ZERO_OPERANDS = args.operands == "zeros"
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import hexmi
    hexmi.lib()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)

    if args.workload == "mfma_peak":
        return run_peak(torch, hexmi, args)
    if args.workload == "issue_slots":
        return run_issue_slots(torch, hexmi, args)
    if args.workload == "lds_patterns":
        return run_lds_patterns(torch, hexmi, args)
    if args.workload == "l2_stream":
        return run_l2_stream(torch, hexmi, args)
    if args.workload == "vendor":
        return run_vendor(torch, hexmi, args)

    wls = make_workloads()
    primary = wls[ALIASES.get(args.workload, args.workload)]
    primary.setup(torch, hexmi)
    m = measure(torch, primary, args.steps, args.warmup, not args.no_graph)
    hot = measure_hot(torch, primary, args.steps, args.warmup, not args.no_graph)
    roof = report(primary, m["ms"])
    unit = roof["unit"]
    line = {
        "metric": "GEMM/attn TFLOP/s + softmax/norm GB/s, % of MI355X roofline, 1 GPU",
        "value": roof["achieved"], "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(m["ms"], 5), "ms_per_step_min": round(m["min"], 5), "ms_per_step_max": round(m["max"], 5),
        "timed_replays": m["replays"], "wall_ms_per_step": round(m["wall"], 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": primary.dtype,
        "data": "synthetic, ALL-ZERO operands (power calibration, not a throughput claim)" if ZERO_OPERANDS else "synthetic",
        "config": {"workload": primary.name, "description": primary.desc,
                   "buffers": "%d rotated sets" % len(primary.sets),
                   "launch": "hip graph replay" if m["graph"] else "direct",
                   "timing": "median of %d replays of the %d-step graph, each replay timed with HIP events"
                             % (m["replays"], args.steps)},
        "roofline": roof,
    }
    if hot is not None:
        line["hot_cache"] = {"ms_per_step": round(hot["ms"], 5), "frac": report(primary, hot["ms"])["frac"],
                             "note": "one buffer set (Infinity-Cache resident where it fits); not the HBM claim"}
    if not args.no_cpu:
        sec, sample = primary.cpu(torch)
        cpu_val = primary.work / sec / (1e9 if primary.bound == "hbm" else 1e12)
        line["cpu_baseline"] = {"value": round(cpu_val, 3), "unit": unit, "cores": cores, "kind": "port",
                                "sample": sample, "ms": round(sec * 1e3, 3)}
    primary.sets = None
    torch.cuda.empty_cache()
    if not args.no_box:
        line["box"] = box_calibration(torch, hexmi)

    if not args.no_suite:
        suite, only = [], [ALIASES.get(n, n) for n in args.only.split(",") if n]
        for name, wl in wls.items():
            if wl is primary or name in ("norms_f16_8192x4096", "copy_64MiB") or (only and name not in only):
                continue
            print("# measuring %s" % name, file=sys.stderr, flush=True)
            wl.setup(torch, hexmi)
            k = steps_for(wl, args.steps)
            wm = measure(torch, wl, k, args.warmup, not args.no_graph)
            whot = measure_hot(torch, wl, k, args.warmup, not args.no_graph)
            entry = entry_for(torch, wl, wm, whot, cores, not args.no_cpu)
            entry["steps"] = k
            if getattr(wl, "step_separate", None) is not None:
                # side figures: the graph forced into one launch, and forced into its separate launches
                own_step = wl.step
                fm = wm
                if getattr(wl, "step_fused", None) is not None:     # the operator's own path may choose either form
                    wl.step = wl.step_fused
                    fm = measure(torch, wl, k, args.warmup, not args.no_graph)
                    entry["one_launch"] = {"ms": round(fm["ms"], 5), "ms_min": round(fm["min"], 5)}
                wl.step = wl.step_separate
                sm = measure(torch, wl, k, args.warmup, not args.no_graph)
                wl.step = own_step
                entry["separate_launches"] = {"launches": wl.launches_separate, "ms": round(sm["ms"], 5),
                                              "ms_min": round(sm["min"], 5),
                                              "speedup_fused": round(sm["ms"] / fm["ms"], 3)}
            if name in ("softmax_f32_4096x1024", "w8a16_m1"):
                entry["direct_launch"] = direct_launch_cost(torch, wl)
            suite.append(entry)
            wl.sets = None
            wl.host = None
            torch.cuda.empty_cache()
        line["suite"] = suite
        by_name = {e["workload"]: e for e in suite}
        targets = []
        for name, want in TARGETS.items():
            e = by_name.get(name)
            if e is not None:
                targets.append({"workload": name, "frac": e["frac"], "frac_best": e["frac_best"], "target": want,
                                "met": bool(e["frac"] >= want)})
        line["targets"] = targets
        line["targets_met"] = "%d of %d" % (sum(t["met"] for t in targets), len(targets))
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
