"""The reference's own oracle calls: PyTorch ops on CPU tensors.

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; never by the product path.

Every end-to-end test of the reference compares its device result with one of
these library calls on the host; they are restated here with the exact
arguments the reference uses so the C oracle can be pinned against them and
so the bench can time "the reference's CPU path" on the host cores.
"""
import torch
import torch.nn.functional as F


def softmax(x):
    """test/python/triton/test_softmax.py:93: F.softmax(x, dim=1, dtype=dtype)."""
    return F.softmax(x, dim=-1, dtype=x.dtype)


def rms_norm(x, weight, eps):
    """test/python/triton/test_rms_norm.py:85-87."""
    return F.rms_norm(x, (x.shape[-1],), weight=weight, eps=eps)


def layer_norm(x, weight, bias, eps):
    """test/python/triton/test_layer_norm.py:111-113."""
    return F.layer_norm(x, (x.shape[-1],), weight=weight, bias=bias, eps=eps)


def matmul(a, b, trans_b=False):
    """test/python/triton/test_matmul.py:90 torch.matmul(A, B); fp32 math on the upcast inputs so that
    the host result does not depend on the CPU's half-precision GEMM."""
    bb = b.float().t() if trans_b else b.float()
    return torch.matmul(a.float(), bb)


def w8a16_matmul(a, w_int8, scales):
    """Closed form of the weight-only int8 matmul (no counterpart in the reference):
    A.float() @ (W.float() * s.float()[:, None]).T."""
    return a.float() @ (w_int8.float() * scales.float()[:, None]).t()


def attention(q, k, v, scale, causal):
    """test/python/triton/test_flash_attention.py:212: F.scaled_dot_product_attention(q, k, v, scale=SCALE)."""
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=causal, scale=scale)


def attention_masked(q, k, v, mask, scale):
    """tm_tensor.attention as torch states it: softmax(QK^T * scale + mask) V with an additive float mask."""
    m = None if mask is None else mask.float()
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=m, scale=scale)
