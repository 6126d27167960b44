"""numpy / ctypes front of the CPU oracle (oracle/hexmi_oracle.c).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; never by the product path.

fp16 arrays are numpy float16; bf16 arrays are numpy uint16 bit patterns
(numpy has no bfloat16) with dtype="bf16" passed explicitly.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")

F32, F16, BF16 = 0, 1, 2


def build(force=False):
    src = os.path.join(_HERE, "hexmi_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def _l():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_f16_to_f32.restype = ctypes.c_float
        _lib.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.oracle_f32_to_f16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    return _lib


def _code(arr, dtype=None):
    if dtype == "bf16":
        assert arr.dtype == np.uint16
        return BF16
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float16:
        return F16
    raise TypeError("oracle: unsupported dtype %s" % arr.dtype)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a):
    return None if a is None else np.ascontiguousarray(a)


_i64, _dbl, _int = ctypes.c_int64, ctypes.c_double, ctypes.c_int


def softmax(x, dtype=None):
    x = _c(x)
    cols = x.shape[-1]
    y = np.empty_like(x)
    _l().oracle_softmax(_ptr(x), _ptr(y), _i64(x.size // max(cols, 1)), _i64(cols), _int(_code(x, dtype)))
    return y


def online_softmax_f32(x, block):
    x = _c(x)
    assert x.dtype == np.float32 and x.ndim == 2
    y = np.empty_like(x)
    _l().oracle_online_softmax_f32(_ptr(x), _ptr(y), _i64(x.shape[0]), _i64(x.shape[1]), _i64(block))
    return y


def rms_norm(x, w, eps, dtype=None):
    x, w = _c(x), _c(w)
    cols = x.shape[-1]
    y = np.empty_like(x)
    _l().oracle_rms_norm(_ptr(x), _ptr(w), _ptr(y), _i64(x.size // max(cols, 1)), _i64(cols), _dbl(eps),
                         _int(_code(x, dtype)))
    return y


def layer_norm(x, w, b, eps, dtype=None):
    """Returns (y, mean, rstd)."""
    x, w, b = _c(x), _c(w), _c(b)
    cols = x.shape[-1]
    rows = x.size // max(cols, 1)
    y = np.empty_like(x)
    mean = np.empty(rows, np.float32)
    rstd = np.empty(rows, np.float32)
    _l().oracle_layer_norm(_ptr(x), _ptr(w), _ptr(b), _ptr(y), _ptr(mean), _ptr(rstd), _i64(rows), _i64(cols),
                           _dbl(eps), _int(_code(x, dtype)))
    return y, mean, rstd


def matmul(a, b, out_dtype=None, trans_b=False, dtype=None):
    """out_dtype: None (same as input), np.float32, np.float16 or 'bf16'."""
    a, b = _c(a), _c(b)
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    code_in = _code(a, dtype)
    if out_dtype is None:
        code_out, c = code_in, np.empty((M, N), a.dtype)
    elif out_dtype == "bf16":
        code_out, c = BF16, np.empty((M, N), np.uint16)
    else:
        c = np.empty((M, N), out_dtype)
        code_out = _code(c)
    _l().oracle_matmul(_ptr(a), _ptr(b), _ptr(c), _i64(M), _i64(N), _i64(K), _int(code_in), _int(code_out),
                       _int(1 if trans_b else 0))
    return c


def linear(a, b, bias=None, residual=None, out_dtype=None, trans_b=False):
    """A op(B) + bias[n] + residual[m, n] with the sums kept in fp32 and ONE rounding to the output type: the linear
    layer whose consumers the reference fuses into the matmul's loop nest
    (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:280-283; the layers of
    test/python/torch-mlir/test_gpt2_block.py). fp16 / fp32 only. Composed of matmul() above (fp32 output) and numpy."""
    out_dtype = out_dtype or a.dtype
    c = matmul(a, b, out_dtype=np.float32, trans_b=trans_b).astype(np.float64)
    if bias is not None:
        c = c + bias.astype(np.float64)[None, :]
    if residual is not None:
        c = c + residual.astype(np.float64)
    return c.astype(np.float32).astype(out_dtype)


def add_matmul_softmax(x, y, z):
    """softmax((x + y) z) over each row: the graph of test/python/torch-mlir/test_add_matmul_softmax.py:19-29
    (torch.add, torch.matmul, torch.softmax(dim=-1)), the sum rounded to the operands' type as torch.add rounds it,
    the product and the softmax in fp32. Composed of matmul() and softmax() above."""
    total = (x.astype(np.float32) + y.astype(np.float32)).astype(x.dtype)
    scores = matmul(total, z, out_dtype=np.float32)
    return softmax(scores).astype(x.dtype)


def dequant_w8(w, scales):
    w, scales = _c(w), _c(scales)
    assert w.dtype == np.int8 and scales.dtype == np.float16
    out = np.empty(w.shape, np.float32)
    _l().oracle_dequant_w8(_ptr(w), _ptr(scales), _ptr(out), _i64(w.shape[0]), _i64(w.shape[1]))
    return out


def matmul_w8a16(a, w, scales):
    a, w, scales = _c(a), _c(w), _c(scales)
    assert a.dtype == np.float16 and w.dtype == np.int8 and scales.dtype == np.float16
    M, K = a.shape
    N = w.shape[0]
    c = np.empty((M, N), np.float16)
    _l().oracle_matmul_w8a16(_ptr(a), _ptr(w), _ptr(scales), _ptr(c), _i64(M), _i64(N), _i64(K))
    return c


def dequant_w8_ex(w, scales, zero_points=None, per_tensor=False):
    """(float(q) - zero_point) * scale with per-channel or per-tensor parameters (zero_points int8 or None)."""
    w, scales = _c(w), _c(scales)
    zp = None if zero_points is None else _c(zero_points)
    assert w.dtype == np.int8 and scales.dtype == np.float16 and (zp is None or zp.dtype == np.int8)
    out = np.empty(w.shape, np.float32)
    _l().oracle_dequant_w8_ex(_ptr(w), _ptr(scales), _ptr(zp) if zp is not None else None, _int(1 if per_tensor else 0),
                              _ptr(out), _i64(w.shape[0]), _i64(w.shape[1]))
    return out


def matmul_w8a16_ex(a, w, scales, zero_points=None, per_tensor=False):
    a, w, scales = _c(a), _c(w), _c(scales)
    zp = None if zero_points is None else _c(zero_points)
    assert a.dtype == np.float16 and w.dtype == np.int8 and scales.dtype == np.float16
    M, K = a.shape
    N = w.shape[0]
    c = np.empty((M, N), np.float16)
    _l().oracle_matmul_w8a16_ex(_ptr(a), _ptr(w), _ptr(scales), _ptr(zp) if zp is not None else None,
                                _int(1 if per_tensor else 0), _ptr(c), _i64(M), _i64(N), _i64(K))
    return c


def pack_w8(w):
    """Fragment-major re-layout of int8 weights [N, K] (K % 64 == 0): tiles of 16 channels x 64 k, tile (t, s) at
    byte ((t*K/64) + s)*1024, lane l = g*16 + r holds W[16t + r][64s + 16g : 64s + 16g + 16]; rows past N are 0.
    A block linearisation in the sense of the reference's weight pre-processing
    (qcom_hexagon_backend/lib/Transforms/PreprocessWeightsForHMXPass.cpp:39-78), written as one index loop."""
    w = _c(w)
    assert w.dtype == np.int8 and w.ndim == 2 and w.shape[1] % 64 == 0
    N, K = w.shape
    T, S = (N + 15) // 16, K // 64
    out = np.zeros(T * 16 * K, np.int8)
    for t in range(T):
        for s_ in range(S):
            for lane in range(64):
                r, g = lane % 16, lane // 16
                row = 16 * t + r
                if row < N:
                    o = ((t * S + s_) * 64 + lane) * 16
                    out[o:o + 16] = w[row, 64 * s_ + 16 * g:64 * s_ + 16 * g + 16]
    return out


def attention(q, k, v, scale, causal, out_dtype=None, dtype=None):
    """q, k, v: [..., S, D]; brute-force softmax(scale*QK^T + mask) V in double."""
    q, k, v = _c(q), _c(k), _c(v)
    S, D = q.shape[-2:]
    ZH = q.size // (S * D)
    code_in = _code(q, dtype)
    if out_dtype is None:
        o, code_out = np.empty_like(q), code_in
    else:
        o = np.empty(q.shape, out_dtype)
        code_out = _code(o)
    _l().oracle_attention(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _i64(ZH), _i64(S), _i64(D), _dbl(scale),
                          _int(1 if causal else 0), _int(code_in), _int(code_out))
    return o


def attention_masked(q, k, v, mask, scale, out_dtype=None, dtype=None):
    """q: [B,Sq,D]; k, v: [B,Skv,D]; mask: [B,Sq,Skv] or None; softmax(scale*QK^T + mask) V in double."""
    q, k, v = _c(q), _c(k), _c(v)
    B, Sq, D = q.shape
    Skv = k.shape[1]
    code_in = _code(q, dtype)
    if mask is not None:
        mask = _c(mask)
        assert mask.shape == (B, Sq, Skv) and mask.dtype == q.dtype
    if out_dtype is None:
        o, code_out = np.empty_like(q), code_in
    else:
        o = np.empty(q.shape, out_dtype)
        code_out = _code(o)
    _l().oracle_attention_masked(_ptr(q), _ptr(k), _ptr(v), _ptr(mask) if mask is not None else None, _ptr(o),
                                 _i64(B), _i64(Sq), _i64(Skv), _i64(D), _dbl(scale), _int(code_in), _int(code_out))
    return o


def attention_online_f32(q, k, v, sm_scale, block_n):
    q, k, v = _c(q), _c(k), _c(v)
    assert q.dtype == np.float32
    S, D = q.shape[-2:]
    o = np.empty_like(q)
    _l().oracle_attention_online_f32(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _i64(q.size // (S * D)), _i64(S), _i64(D),
                                     ctypes.c_float(sm_scale), _i64(block_n))
    return o


UNARY_OPS = {"gelu_tanh": 0, "silu": 1, "rsqrt": 2, "sin": 3, "cos": 4, "exp": 5}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def unary(op, x, dtype=None):
    x = _c(x)
    y = np.empty_like(x)
    _l().oracle_unary(_int(UNARY_OPS[op]), _ptr(x), _ptr(y), _i64(x.size), _int(_code(x, dtype)))
    return y


def binary(op, a, b, dtype=None):
    a, b = _c(a), _c(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    y = np.empty_like(a)
    _l().oracle_binary(_int(BINARY_OPS[op]), _ptr(a), _ptr(b), _ptr(y), _i64(a.size), _int(_code(a, dtype)))
    return y


def block_sum(x, block, dtype=None):
    x = _c(x).reshape(-1)
    out = np.empty(((x.size + block - 1) // block,), x.dtype)
    _l().oracle_block_sum(_ptr(x), _ptr(out), _i64(x.size), _i64(block), _int(_code(x, dtype)))
    return out


def rope(x, theta, dtype=None):
    """x: [batch, seq, heads, feat]."""
    x = _c(x)
    B, L, H, D = x.shape
    y = np.empty_like(x)
    _l().oracle_rope(_ptr(x), _ptr(y), _i64(B), _i64(L), _i64(H), _i64(D), _dbl(theta), _int(_code(x, dtype)))
    return y


def f32_to_f16_bits(v):
    return _l().oracle_f32_to_f16(ctypes.c_float(v))


def f16_bits_to_f32(h):
    return _l().oracle_f16_to_f32(ctypes.c_uint16(h))


def f32_to_bf16_bits(v):
    return _l().oracle_f32_to_bf16(ctypes.c_float(v))
