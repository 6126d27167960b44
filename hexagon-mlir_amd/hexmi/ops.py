"""Tensor-in / tensor-out operators over libhexmi.so.

Every operator is registered as a PyTorch custom op (`torch.ops.hexmi.*`,
CUDA/HIP dispatch key only) whose implementation hands device pointers and the
current HIP stream to the C ABI. The public functions below add what the
reference's launcher does around a kernel: host tensors are accepted, staged
to the GPU, and results are written back into the caller's `out` tensor in
place (qcom_hexagon_backend/backend/triton_hexagon_launcher.py:716-728 copies
device results back into the tensors the user passed).

There is no CPU implementation: without a GPU or without libhexmi.so these
functions raise.
"""
import math

import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.int8: _lib.I8}


def _dt(t):
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError("hexmi: unsupported dtype %s" % t.dtype) from None


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_RAW_DEVICE = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current device's current HIP stream as an integer handle (the raw getters skip building a
    torch.cuda.Stream object per call, which costs more than a ctypes call)."""
    if _RAW_STREAM is not None and _RAW_DEVICE is not None:
        return _RAW_STREAM(_RAW_DEVICE())
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device):
    """Context that makes `device` current for the launch; free when it already is (the usual case: entering
    torch.cuda.device() costs more than the shortest kernels here run)."""
    if device.index is None or device.index == (_RAW_DEVICE() if _RAW_DEVICE is not None
                                                else torch.cuda.current_device()):
        return _NO_SWITCH
    return torch.cuda.device(device)


# --------------------------------------------------------------------------
# custom-op registration (schema: inputs..., Tensor(a!) out) -> ()
# --------------------------------------------------------------------------
_LIBDEF = torch.library.Library("hexmi", "DEF")
_LIBDEF.define("softmax(Tensor x, Tensor(a!) out) -> ()")
_LIBDEF.define("rms_norm(Tensor x, Tensor? weight, float eps, Tensor(a!) out) -> ()")
_LIBDEF.define("layer_norm(Tensor x, Tensor? weight, Tensor? bias, float eps, Tensor(a!) out, "
               "Tensor(b!)? mean, Tensor(c!)? rstd) -> ()")
_LIBDEF.define("matmul(Tensor a, Tensor b, bool trans_b, Tensor(a!) out) -> ()")
_LIBDEF.define("linear(Tensor a, Tensor b, Tensor? bias, Tensor? residual, bool trans_b, Tensor(a!) out) -> ()")
_LIBDEF.define("add_matmul_softmax(Tensor x, Tensor y, Tensor z, Tensor(a!) out) -> ()")
_LIBDEF.define("w8a16_matmul(Tensor a, Tensor w, Tensor scales, Tensor(a!) out) -> ()")
_LIBDEF.define("dequant_w8(Tensor w, Tensor scales, Tensor(a!) out) -> ()")
_LIBDEF.define("pack_w8(Tensor w, Tensor(a!) out) -> ()")
_LIBDEF.define("w8a16_matmul_packed(Tensor a, Tensor wp, Tensor scales, Tensor(a!) out) -> ()")
_LIBDEF.define("flash_attention(Tensor q, Tensor k, Tensor v, float sm_scale, bool causal, Tensor(a!) out) -> ()")
_LIBDEF.define("unary(int op, Tensor x, Tensor(a!) out) -> ()")
_LIBDEF.define("binary(int op, Tensor a, Tensor b, Tensor(a!) out) -> ()")
_LIBDEF.define("block_sum(Tensor x, int block, Tensor(a!) out) -> ()")
_LIBDEF.define("rope(Tensor x, float theta, Tensor(a!) out) -> ()")
_LIBDEF.define("attention(Tensor q, Tensor k, Tensor v, Tensor? mask, float sm_scale, Tensor(a!) out) -> ()")


def _row_workspace(rows, cols, block_cols, x):
    """Scratch for the row operators' split form (rows cut into column blocks that several workgroups reduce): the
    library says how much the shape takes, 0 when its single-pass kernels run anyway."""
    need = _lib.lib().hexmi_row_workspace(rows, cols, block_cols, _dt(x))
    return (torch.empty(need, dtype=torch.uint8, device=x.device), need) if need else (None, 0)


def _row_geometry(x, out, rows, cols):
    """(rows, cols, ld_x, ld_out): 2-D tensors whose rows are contiguous may be strided views (ld = row stride);
    anything else is contiguous with rows and cols given."""
    if rows is None:
        rows, cols = x.shape
        return rows, cols, x.stride(0), out.stride(0)
    return rows, cols, cols, cols


def _softmax_impl(x, out, rows=None, cols=None, block_cols=0):
    """x, out: [rows, cols]; or contiguous tensors of any rank with rows and cols given (no view objects built)."""
    rows, cols, ldx, ldo = _row_geometry(x, out, rows, cols)
    with _on(x.device):
        ws, need = _row_workspace(rows, cols, block_cols, x)
        _lib.check(_lib.lib().hexmi_softmax_ws(_p(x), _p(out), rows, cols, ldx, ldo, block_cols, _dt(x), _p(ws), need,
                                               _stream()), "hexmi_softmax_ws")


def _rms_norm_impl(x, weight, eps, out, rows=None, cols=None, block_cols=0):
    rows, cols, ldx, ldo = _row_geometry(x, out, rows, cols)
    with _on(x.device):
        ws, need = _row_workspace(rows, cols, block_cols, x)
        _lib.check(_lib.lib().hexmi_rms_norm_ws(_p(x), _p(weight), _p(out), rows, cols, ldx, ldo, eps, block_cols,
                                                _dt(x), _p(ws), need, _stream()), "hexmi_rms_norm_ws")


def _layer_norm_impl(x, weight, bias, eps, out, mean, rstd, rows=None, cols=None, block_cols=0):
    rows, cols, ldx, ldo = _row_geometry(x, out, rows, cols)
    with _on(x.device):
        ws, need = _row_workspace(rows, cols, block_cols, x)
        _lib.check(_lib.lib().hexmi_layer_norm_ws(_p(x), _p(weight), _p(bias), _p(out), _p(mean), _p(rstd), rows, cols,
                                                  ldx, ldo, eps, block_cols, _dt(x), _p(ws), need, _stream()),
                   "hexmi_layer_norm_ws")


def _matmul_impl(a, b, trans_b, out):
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    with _on(a.device):
        _lib.check(_lib.lib().hexmi_gemm(M, N, K, _p(a), a.stride(0), _p(b), b.stride(0), _p(out), out.stride(0),
                                         _dt(a), _dt(out), 1 if trans_b else 0, _stream()), "hexmi_gemm")


def _linear_impl(a, b, bias, residual, trans_b, out):
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    with _on(a.device):
        _lib.check(_lib.lib().hexmi_gemm_ex(M, N, K, _p(a), a.stride(0), _p(b), b.stride(0), _p(out), out.stride(0),
                                            _p(bias), _p(residual), residual.stride(0) if residual is not None else 0,
                                            _dt(a), _dt(out), 1 if trans_b else 0, _stream()), "hexmi_gemm_ex")


def _add_matmul_softmax_impl(x, y, z, out):
    M, K = x.shape
    N = z.shape[1]
    with _on(x.device):
        _lib.check(_lib.lib().hexmi_add_matmul_softmax(M, N, K, _p(x), x.stride(0), _p(y), y.stride(0), _p(z),
                                                       z.stride(0), _p(out), out.stride(0), _dt(x), _stream()),
                   "hexmi_add_matmul_softmax")


_W8_WORKSPACES = {}          # (device index, stream) -> uint8 tensor, grown on demand


def _w8a16_impl(a, w, scales, out):
    M, K = a.shape
    N = w.shape[0]
    with _on(a.device):
        # shapes the library sums over several K parts need fp32 scratch for the partial tiles; one buffer per device
        # and stream is kept and reused (calls on one stream are ordered, so they may share it)
        need = _lib.lib().hexmi_gemm_w8a16_workspace(M, N, K)
        ws = None
        if need:
            key = (a.device.index, _stream())
            ws = _W8_WORKSPACES.get(key)
            if ws is None or ws.numel() < need:
                ws = torch.empty(need, dtype=torch.uint8, device=a.device)
                _W8_WORKSPACES[key] = ws
        _lib.check(_lib.lib().hexmi_gemm_w8a16_ws(M, N, K, _p(a), _p(w), _p(scales), _p(out), _p(ws),
                                                  ws.numel() if ws is not None else 0, _stream()),
                   "hexmi_gemm_w8a16_ws")


def _pack_impl(w, out):
    N, K = w.shape
    with _on(w.device):
        _lib.check(_lib.lib().hexmi_pack_w8(N, K, _p(w), _p(out), _stream()), "hexmi_pack_w8")


def _w8a16_packed_impl(a, wp, scales, out):
    M, K = a.shape
    N = scales.shape[0]
    with _on(a.device):
        _lib.check(_lib.lib().hexmi_gemm_w8a16_packed(M, N, K, _p(a), _p(wp), _p(scales), _p(out), _stream()),
                   "hexmi_gemm_w8a16_packed")


def _dequant_impl(w, scales, out):
    N, K = w.shape
    with _on(w.device):
        _lib.check(_lib.lib().hexmi_dequant_w8(N, K, _p(w), _p(scales), _p(out), _stream()), "hexmi_dequant_w8")


def _flash_impl(q, k, v, sm_scale, causal, out):
    Z, H, S, D = q.shape
    with _on(q.device):
        _lib.check(_lib.lib().hexmi_flash_attn_fwd(_p(q), _p(k), _p(v), _p(out), Z, H, S, D, sm_scale,
                                                   1 if causal else 0, _dt(q), _dt(out), _stream()),
                   "hexmi_flash_attn_fwd")


def _attention_impl(q, k, v, mask, sm_scale, out):
    B, Sq, D = q.shape
    Skv = k.shape[1]
    with _on(q.device):
        _lib.check(_lib.lib().hexmi_attention(_p(q), _p(k), _p(v), _p(mask), _p(out), B, Sq, Skv, D, sm_scale,
                                              _dt(q), _dt(out), _stream()), "hexmi_attention")


def _unary_impl(op, x, out):
    with _on(x.device):
        _lib.check(_lib.lib().hexmi_unary(op, _p(x), _p(out), x.numel(), _dt(x), _stream()), "hexmi_unary")


def _binary_impl(op, a, b, out):
    with _on(a.device):
        _lib.check(_lib.lib().hexmi_binary(op, _p(a), _p(b), _p(out), a.numel(), _dt(a), _stream()), "hexmi_binary")


def _block_sum_impl(x, block, out):
    n = x.numel()
    need = _lib.lib().hexmi_block_sum_workspace(n, block, _dt(x))
    # huge programs (the reference test sums 2^20 elements in one) are summed in two passes over the whole chip
    # when the library is handed scratch for its fp32 partial sums
    ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
    with _on(x.device):
        _lib.check(_lib.lib().hexmi_block_sum_ws(_p(x), _p(out), n, block, _dt(x), _p(ws), need, _stream()),
                   "hexmi_block_sum_ws")


def _rope_impl(x, theta, out):
    B, L, H, D = x.shape
    with _on(x.device):
        _lib.check(_lib.lib().hexmi_rope(_p(x), _p(out), B, L, H, D, theta, _dt(x), _stream()), "hexmi_rope")


for _name, _fn in (("softmax", _softmax_impl), ("rms_norm", _rms_norm_impl), ("layer_norm", _layer_norm_impl),
                   ("matmul", _matmul_impl), ("linear", _linear_impl), ("add_matmul_softmax", _add_matmul_softmax_impl),
                   ("w8a16_matmul", _w8a16_impl), ("dequant_w8", _dequant_impl), ("pack_w8", _pack_impl),
                   ("w8a16_matmul_packed", _w8a16_packed_impl),
                   ("flash_attention", _flash_impl), ("attention", _attention_impl),
                   ("unary", _unary_impl), ("binary", _binary_impl), ("block_sum", _block_sum_impl),
                   ("rope", _rope_impl)):
    _LIBDEF.impl(_name, _fn, "CUDA")


# --------------------------------------------------------------------------
# staging helpers
# --------------------------------------------------------------------------
def _device():
    if not torch.cuda.is_available():
        raise RuntimeError("hexmi needs a GPU (gfx950); there is no CPU path")
    _lib.lib()
    return torch.device("cuda", torch.cuda.current_device())


def _stage(t, dev):
    """Contiguous device copy (or the tensor itself when it already is one)."""
    if t is None:
        return None
    if t.device.type != "cuda":
        t = t.to(dev, non_blocking=False)
    return t if t.is_contiguous() else t.contiguous()


def _finish(result, out):
    """Write `result` (device) into the caller's `out` if they are different tensors."""
    if out is None:
        return result
    if out.data_ptr() != result.data_ptr() or out.device != result.device:
        out.copy_(result)
    return out


def _out_like(out, shape, dtype, dev):
    """Device tensor to compute into: `out` itself when usable, else a fresh one."""
    if out is not None:
        if tuple(out.shape) != tuple(shape):
            raise ValueError("hexmi: out has shape %s, expected %s" % (tuple(out.shape), tuple(shape)))
        if out.dtype != dtype:
            raise TypeError("hexmi: out has dtype %s, expected %s" % (out.dtype, dtype))
        if out.device.type == "cuda" and out.is_contiguous():
            return out
    return torch.empty(shape, dtype=dtype, device=dev)


# --------------------------------------------------------------------------
# public operators. They call the implementations above directly: the same code `torch.ops.hexmi.*` runs, without
# the dispatcher's round trip into Python (several microseconds, more than the shortest kernels here take).
# A caller that traces a model (torch.compile, FakeTensor propagation) needs the operators to appear as
# `torch.ops.hexmi.*` nodes: `through_dispatcher(True)` routes the operators that have a registered schema through
# the dispatcher (2-D operands, no column blocks; anything else keeps the direct call).
# --------------------------------------------------------------------------
_THROUGH_DISPATCHER = False


def through_dispatcher(enable=True):
    """Route softmax / rms_norm / layer_norm / matmul / w8a16_matmul / flash_attention through `torch.ops.hexmi.*`
    (visible to tracing) instead of calling the library directly. Returns the previous setting."""
    global _THROUGH_DISPATCHER
    previous, _THROUGH_DISPATCHER = _THROUGH_DISPATCHER, bool(enable)
    return previous


def _run(name, impl, simple, *args):
    """impl(*args) directly, or torch.ops.hexmi.<name>(*simple) when tracing asked for the dispatcher and the call
    has the registered operator's form (simple is not None)."""
    if _THROUGH_DISPATCHER and simple is not None:
        getattr(torch.ops.hexmi, name)(*simple)
    else:
        impl(*args)


def _row_strided(t):
    """A 2-D device tensor whose rows are contiguous but not adjacent (a column slice, a padded buffer): the row
    operators read and write it in place through its row stride, as the reference's kernels take a memref with
    strides (test/utils/dsp/include/common.h:15-21)."""
    return (t is not None and t.device.type == "cuda" and t.dim() == 2 and t.stride(1) == 1
            and t.stride(0) >= t.shape[1] and not t.is_contiguous())


def _row_operands(x, out, dev):
    """(x on the device, tensor to compute into, rows, cols) with rows / cols None when both are 2-D strided views."""
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    if _row_strided(x) or (_row_strided(out) and x.dim() == 2):
        xd = x if x.device.type == "cuda" and x.dim() == 2 and x.stride(1) == 1 else _stage(x, dev)
        if out is not None and (tuple(out.shape) != tuple(x.shape) or out.dtype != x.dtype):
            raise ValueError("hexmi: out must have the shape and dtype of x")
        od = out if (out is not None and out.device.type == "cuda" and out.stride(1) == 1) else torch.empty_like(xd, memory_format=torch.contiguous_format)
        return xd, od, None, None
    return _stage(x, dev), _out_like(out, x.shape, x.dtype, dev), rows, cols


def softmax(x, out=None, dim=-1, block_cols=0):
    """Softmax over the last dimension (`F.softmax(x, dim=1)` of
    test/python/triton/test_softmax.py:93 for 2-D input). block_cols > 0: the two-phase (online) form of
    test/python/triton/test_online_softmax.py:31-81 over column blocks of that size."""
    if dim not in (-1, x.dim() - 1):
        raise ValueError("hexmi.softmax reduces over the last dimension only")
    if x.dim() < 1:
        raise ValueError("hexmi.softmax needs at least 1 dimension")
    dev = _device() if x.device.type != "cuda" else x.device
    xd, od, rows, cols = _row_operands(x, out, dev)
    _run("softmax", _softmax_impl, (xd, od) if xd.dim() == 2 and not block_cols else None, xd, od, rows, cols, int(block_cols))
    return _finish(od, out)


def rms_norm(x, weight=None, eps=1e-5, out=None, block_cols=0):
    """`F.rms_norm(x, (C,), weight, eps)` (test/python/triton/test_rms_norm.py:85-87)."""
    dev = _device() if x.device.type != "cuda" else x.device
    cols = x.shape[-1]
    if weight is not None and (weight.shape != (cols,) or weight.dtype != x.dtype):
        raise ValueError("hexmi.rms_norm: weight must be [%d] of %s" % (cols, x.dtype))
    xd, od, rows, c = _row_operands(x, out, dev)
    wd = _stage(weight, dev)
    _run("rms_norm", _rms_norm_impl, (xd, wd, float(eps), od) if xd.dim() == 2 and not block_cols else None,
         xd, wd, float(eps), od, rows, c, int(block_cols))
    return _finish(od, out)


def layer_norm(x, weight=None, bias=None, eps=1e-5, out=None, mean=None, rstd=None, block_cols=0):
    """`F.layer_norm(x, (C,), weight, bias, eps)` (test/python/triton/test_layer_norm.py:111-113);
    `mean` / `rstd` (fp32, one per row) are filled when given, as the reference kernel does."""
    dev = _device() if x.device.type != "cuda" else x.device
    cols = x.shape[-1]
    nrows = x.numel() // max(cols, 1)
    for name, t in (("weight", weight), ("bias", bias)):
        if t is not None and (t.shape != (cols,) or t.dtype != x.dtype):
            raise ValueError("hexmi.layer_norm: %s must be [%d] of %s" % (name, cols, x.dtype))
    xd, od, rows, c = _row_operands(x, out, dev)
    wd, bd = _stage(weight, dev), _stage(bias, dev)
    md = None if mean is None else _out_like(mean if mean.dtype == torch.float32 else None, (nrows,), torch.float32, dev)
    rd = None if rstd is None else _out_like(rstd if rstd.dtype == torch.float32 else None, (nrows,), torch.float32, dev)
    _run("layer_norm", _layer_norm_impl, (xd, wd, bd, float(eps), od, md, rd) if xd.dim() == 2 and not block_cols else None,
         xd, wd, bd, float(eps), od, md, rd, rows, c, int(block_cols))
    if mean is not None:
        _finish(md, mean)
    if rstd is not None:
        _finish(rd, rstd)
    return _finish(od, out)


def matmul(a, b, out=None, out_dtype=None, trans_b=False, bias=None, residual=None):
    """C = A @ B (or A @ B.T when trans_b), fp16/bf16 inputs with fp32 accumulation on the matrix cores, or fp32
    inputs multiplied in fp32. out_dtype: the input dtype (default) or torch.float32
    (test/python/triton/test_matmul.py:35-91; docs/tutorials/triton/matmul_hexkl.md:61-111).
    bias [N] and residual [M,N] (of the output dtype) are added to the fp32 sums inside the GEMM kernel, the way the
    reference's fusion pass pulls the consumers of a matmul into its loop nest
    (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:280-283): C = A @ B + bias + residual
    with one rounding and no extra launch."""
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("hexmi.matmul takes 2-D tensors")
    if a.dtype != b.dtype or a.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError("hexmi.matmul: A and B must both be float16, both bfloat16 or both float32")
    if a.dtype == torch.float32 and (out_dtype or (out.dtype if out is not None else torch.float32)) != torch.float32:
        raise TypeError("hexmi.matmul: float32 operands give a float32 result")
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != K:
        raise ValueError("hexmi.matmul: inner dimensions differ: %s x %s" % (tuple(a.shape), tuple(b.shape)))
    if out_dtype is None:
        out_dtype = out.dtype if out is not None else a.dtype
    if bias is not None and (bias.shape != (N,) or bias.dtype != out_dtype):
        raise ValueError("hexmi.matmul: bias must be [N] of the output dtype")
    if residual is not None and (residual.shape != (M, N) or residual.dtype != out_dtype):
        raise ValueError("hexmi.matmul: residual must be [M,N] of the output dtype")
    dev = _device() if a.device.type != "cuda" else a.device
    ad, bd = _stage(a, dev), _stage(b, dev)
    od = _out_like(out, (M, N), out_dtype, dev)
    if bias is None and residual is None:
        _run("matmul", _matmul_impl, (ad, bd, bool(trans_b), od), ad, bd, bool(trans_b), od)
    else:
        _linear_impl(ad, bd, _stage(bias, dev), _stage(residual, dev), bool(trans_b), od)
    return _finish(od, out)


def pack_weight(w):
    """One-time re-layout of a constant 16-bit weight [K,N] into the K-contiguous form [N,K] the GEMM streams fastest;
    multiply with `matmul(a, packed, trans_b=True)`. The analogue of the reference folding the transpose of a
    constant weight at compile time (qcom_hexagon_backend/lib/Transforms/FoldResourceTransposePass.cpp:21-110)."""
    if w.dim() != 2 or w.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("hexmi.pack_weight: expected a 2-D float16 or bfloat16 tensor")
    dev = _device() if w.device.type != "cuda" else w.device
    wd = _stage(w, dev)
    rows, cols = wd.shape
    out = torch.empty((cols, rows), dtype=w.dtype, device=dev)
    with _on(dev):
        _lib.check(_lib.lib().hexmi_transpose16(rows, cols, _p(wd), wd.stride(0), _p(out), out.stride(0), _stream()),
                   "hexmi_transpose16")
    return out


def _quant_params(name, w_int8, scales, zero_points):
    """Checks the parameters of `f = (float(q) - zero_point) * scale`; returns per_tensor (one scale, and one zero
    point, for the whole tensor) against per output channel."""
    if w_int8.dtype != torch.int8 or scales.dtype != torch.float16:
        raise TypeError("hexmi.%s: expected int8 weights, fp16 scales" % name)
    if w_int8.dim() != 2 or scales.dim() != 1 or scales.shape[0] not in (1, w_int8.shape[0]):
        raise ValueError("hexmi.%s: shapes W[N,K] and scales[N] (per channel) or scales[1] (per tensor) required" % name)
    per_tensor = scales.shape[0] == 1 and w_int8.shape[0] != 1
    if zero_points is not None:
        if zero_points.dtype != torch.int8:
            raise TypeError("hexmi.%s: zero points are int8" % name)
        if zero_points.shape != scales.shape:
            raise ValueError("hexmi.%s: zero_points must have the shape of scales" % name)
    return per_tensor


def w8a16_matmul(a, w_int8, scales, out=None, zero_points=None):
    """C[m,n] = sum_k A[m,k] * ((W[n,k] - zero_points[n]) * scales[n]); A fp16 [M,K], W int8 [N,K], scales fp16 [N]
    (or [1]: one scale and zero point for the tensor), zero_points int8 or None (symmetric)."""
    if a.dtype != torch.float16:
        raise TypeError("hexmi.w8a16_matmul: expected fp16 activations, int8 weights, fp16 scales")
    if w_int8.dtype != torch.int8 or scales.dtype != torch.float16:
        raise TypeError("hexmi.w8a16_matmul: expected fp16 activations, int8 weights, fp16 scales")
    if a.dim() != 2 or w_int8.dim() != 2 or a.shape[1] != w_int8.shape[1]:
        raise ValueError("hexmi.w8a16_matmul: shapes A[M,K], W[N,K], scales[N] required")
    per_tensor = _quant_params("w8a16_matmul", w_int8, scales, zero_points)
    dev = _device() if a.device.type != "cuda" else a.device
    ad, wd, sd = _stage(a, dev), _stage(w_int8, dev), _stage(scales, dev)
    od = _out_like(out, (a.shape[0], w_int8.shape[0]), torch.float16, dev)
    if zero_points is None and not per_tensor:
        _run("w8a16_matmul", _w8a16_impl, (ad, wd, sd, od), ad, wd, sd, od)
    else:
        zd = _stage(zero_points, dev)
        M, K = ad.shape
        with _on(ad.device):
            _lib.check(_lib.lib().hexmi_gemm_w8a16_ex(M, wd.shape[0], K, _p(ad), _p(wd), _p(sd), _p(zd),
                                                      1 if per_tensor else 0, _p(od), _stream()), "hexmi_gemm_w8a16_ex")
    return _finish(od, out)


def pack_w8(w_int8):
    """One-time re-layout of int8 weights [N,K] (K % 64 == 0) into the fragment-major order `w8a16_matmul_packed`
    reads (flat int8 tensor of ceil(N/16)*16*K bytes); the analogue of the reference's constant-weight
    pre-processing (qcom_hexagon_backend/lib/Transforms/PreprocessWeightsForHMXPass.cpp:39-117)."""
    if w_int8.dtype != torch.int8 or w_int8.dim() != 2:
        raise TypeError("hexmi.pack_w8: expected an int8 [N,K] tensor")
    N, K = w_int8.shape
    if K % 64 != 0:
        raise ValueError("hexmi.pack_w8: K must be a multiple of 64")
    dev = _device() if w_int8.device.type != "cuda" else w_int8.device
    wd = _stage(w_int8, dev)
    out = torch.empty(((N + 15) // 16) * 16 * K, dtype=torch.int8, device=dev)
    _pack_impl(wd, out)
    return out


def w8a16_matmul_packed(a, w_packed, scales, out=None):
    """`w8a16_matmul` on weights packed by `pack_w8` (N = len(scales)). Same result bit for bit for 3 <= M <= 8
    (the same kernel); for other M `w8a16_matmul` uses kernels that sum in another order (one fp16 ulp)."""
    if a.dtype != torch.float16 or w_packed.dtype != torch.int8 or scales.dtype != torch.float16:
        raise TypeError("hexmi.w8a16_matmul_packed: expected fp16 activations, packed int8 weights, fp16 scales")
    if a.dim() != 2 or scales.dim() != 1:
        raise ValueError("hexmi.w8a16_matmul_packed: shapes A[M,K], scales[N] required")
    M, K = a.shape
    N = scales.shape[0]
    if w_packed.numel() != ((N + 15) // 16) * 16 * K:
        raise ValueError("hexmi.w8a16_matmul_packed: packed weights do not match N=%d, K=%d" % (N, K))
    dev = _device() if a.device.type != "cuda" else a.device
    ad, wd, sd = _stage(a, dev), _stage(w_packed, dev), _stage(scales, dev)
    od = _out_like(out, (M, N), torch.float16, dev)
    _w8a16_packed_impl(ad, wd, sd, od)
    return _finish(od, out)


def dequant_w8(w_int8, scales, out=None, zero_points=None):
    """fp32 [N,K] = (float(W[n,k]) - zero_points[n]) * float(scales[n]) (the dequantisation the fused kernel applies;
    scales / zero_points of one element: per tensor)."""
    per_tensor = _quant_params("dequant_w8", w_int8, scales, zero_points)
    dev = _device() if w_int8.device.type != "cuda" else w_int8.device
    wd, sd = _stage(w_int8, dev), _stage(scales, dev)
    od = _out_like(out, w_int8.shape, torch.float32, dev)
    if zero_points is None and not per_tensor:
        _dequant_impl(wd, sd, od)
    else:
        zd = _stage(zero_points, dev)
        with _on(wd.device):
            _lib.check(_lib.lib().hexmi_dequant_w8_ex(wd.shape[0], wd.shape[1], _p(wd), _p(sd), _p(zd),
                                                      1 if per_tensor else 0, _p(od), _stream()), "hexmi_dequant_w8_ex")
    return _finish(od, out)


def flash_attention(q, k, v, sm_scale=None, causal=False, out=None, out_dtype=None):
    """softmax(sm_scale * Q K^T [+causal]) V for [Z,H,S,D] tensors
    (`F.scaled_dot_product_attention(q, k, v, scale=...)`, test/python/triton/test_flash_attention.py:212)."""
    if q.dim() != 4 or q.shape != k.shape or q.shape != v.shape:
        raise ValueError("hexmi.flash_attention: q, k, v must share one [Z,H,S,D] shape")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("hexmi.flash_attention: q, k, v dtypes differ")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    if out_dtype is None:
        out_dtype = out.dtype if out is not None else q.dtype
    dev = _device() if q.device.type != "cuda" else q.device
    qd, kd, vd = _stage(q, dev), _stage(k, dev), _stage(v, dev)
    od = _out_like(out, q.shape, out_dtype, dev)
    _run("flash_attention", _flash_impl, (qd, kd, vd, float(sm_scale), bool(causal), od), qd, kd, vd, float(sm_scale), bool(causal), od)
    return _finish(od, out)


def attention(q, k, v, mask=None, sm_scale=None, out=None, out_dtype=None):
    """tm_tensor.attention: softmax(Q K^T / sqrt(d) + mask) V for q [B,Sq,D], k / v [B,Skv,D] and an additive
    mask [B,Sq,Skv] (or None) (include/hexagon/Dialect/TmTensor/IR/TmTensorOps.td:28-56,
    lib/Transforms/LowerTmTensor.cpp:70-235); `F.scaled_dot_product_attention(q, k, v, attn_mask=mask)`."""
    if q.dim() != 3 or k.dim() != 3 or v.shape != k.shape or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise ValueError("hexmi.attention: q [B,Sq,D], k and v [B,Skv,D]")
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("hexmi.attention: q, k, v dtypes differ")
    B, Sq, D = q.shape
    Skv = k.shape[1]
    if mask is not None and (tuple(mask.shape) != (B, Sq, Skv) or mask.dtype != q.dtype):
        raise ValueError("hexmi.attention: mask must be [%d,%d,%d] of %s" % (B, Sq, Skv, q.dtype))
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    if out_dtype is None:
        out_dtype = out.dtype if out is not None else q.dtype
    dev = _device() if q.device.type != "cuda" else q.device
    qd, kd, vd, md = _stage(q, dev), _stage(k, dev), _stage(v, dev), _stage(mask, dev)
    od = _out_like(out, q.shape, out_dtype, dev)
    _attention_impl(qd, kd, vd, md, float(sm_scale), od)
    return _finish(od, out)


UNARY_OPS = {"gelu_tanh": 0, "silu": 1, "rsqrt": 2, "sin": 3, "cos": 4, "exp": 5}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def unary(op, x, out=None):
    """Element-wise `op` in UNARY_OPS ("gelu_tanh": test/python/triton/test_gelu.py:43-54, "silu": test_silu.py:43-52,
    "rsqrt": test_rsqrt.py:20-24, "sin" / "cos": test_math_ops.py:25-38, "exp")."""
    if op not in UNARY_OPS:
        raise ValueError("hexmi.unary: unknown op %r" % (op,))
    dev = _device() if x.device.type != "cuda" else x.device
    xd = _stage(x, dev)
    od = _out_like(out, x.shape, x.dtype, dev)
    _unary_impl(UNARY_OPS[op], xd, od)
    return _finish(od, out)


def gelu(x, out=None):
    """`F.gelu(x, approximate="tanh")` (test/python/triton/test_gelu.py:73)."""
    return unary("gelu_tanh", x, out)


def silu(x, out=None):
    """`F.silu(x)` (test/python/triton/test_silu.py:69)."""
    return unary("silu", x, out)


def binary(op, a, b, out=None):
    """Element-wise a (op) b for same-shape tensors, op in BINARY_OPS (test/python/triton/test_vec_add.py,
    test_vec_div_2d.py:21-55)."""
    if op not in BINARY_OPS:
        raise ValueError("hexmi.binary: unknown op %r" % (op,))
    if a.shape != b.shape or a.dtype != b.dtype:
        raise ValueError("hexmi.binary: operands must share shape and dtype")
    dev = _device() if a.device.type != "cuda" else a.device
    ad, bd = _stage(a, dev), _stage(b, dev)
    od = _out_like(out, a.shape, a.dtype, dev)
    _binary_impl(BINARY_OPS[op], ad, bd, od)
    return _finish(od, out)


def block_sum(x, block=None, out=None):
    """out[p] = sum of the p-th run of `block` elements of x (flattened); block=None sums everything into out[0]
    (`torch.sum(x)`, test/python/triton/test_sum.py:30-47)."""
    n = x.numel()
    if block is None:
        block = max(n, 1)
    if block < 1:
        raise ValueError("hexmi.block_sum: block must be positive")
    programs = (n + block - 1) // block
    dev = _device() if x.device.type != "cuda" else x.device
    xd = _stage(x, dev).reshape(-1)
    od = _out_like(out, (programs,), x.dtype, dev)
    _block_sum_impl(xd, int(block), od)
    return _finish(od, out)


def rope(x, theta=10000.0, out=None):
    """Rotary embedding of x [batch, seq, heads, features] over adjacent feature pairs
    (`rope_reference_pytorch`, test/python/triton/test_rope.py:60-95)."""
    if x.dim() != 4 or x.shape[-1] % 2 != 0:
        raise ValueError("hexmi.rope: x must be [batch, seq, heads, features] with an even feature count")
    dev = _device() if x.device.type != "cuda" else x.device
    xd = _stage(x, dev)
    od = _out_like(out, x.shape, x.dtype, dev)
    _rope_impl(xd, float(theta), od)
    return _finish(od, out)


# Above this much multiply-add work the one-launch kernel (32 rows per workgroup, so few workgroups on small
# problems, and scalar guarded copies) loses to add -> tiled GEMM -> softmax: measured 5.9 us against 6.2 us at
# 32x32x32, 29 us against 10 us at 512x512x64. Below it the two saved launches and round trips win.
_FUSED_MAX_MACS = 1 << 20


def add_matmul_softmax(x, y, z, out=None, fused=None):
    """softmax((x + y) @ z, dim=-1): the graph of test/python/torch-mlir/test_add_matmul_softmax.py:19-29, which the
    reference compiles into one fused kernel. One launch (`hexmi_add_matmul_softmax`) when the result has at most
    1024 columns and the product is small; otherwise the three kernels run back to back on one stream.
    fused=True / False forces one or the other."""
    if x.shape != y.shape or x.dim() != 2 or z.dim() != 2 or x.shape[1] != z.shape[0]:
        raise ValueError("hexmi.add_matmul_softmax: x, y [M,K] and z [K,N] required")
    if not (x.dtype == y.dtype == z.dtype) or x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError("hexmi.add_matmul_softmax: x, y, z must share one of float16, bfloat16, float32")
    dev = _device() if x.device.type != "cuda" else x.device
    M, K = x.shape
    N = z.shape[1]
    fits = 0 < N <= _lib.lib().hexmi_add_matmul_softmax_max_n()
    if fused is None:
        fused = fits and M * N * K <= _FUSED_MAX_MACS
    if fused:
        if not fits:
            raise ValueError("hexmi.add_matmul_softmax: the one-launch kernel takes at most 1024 columns")
        od = _out_like(out, (M, N), x.dtype, dev)
        _add_matmul_softmax_impl(_stage(x, dev), _stage(y, dev), _stage(z, dev), od)
        return _finish(od, out)
    total = binary("add", _stage(x, dev), _stage(y, dev))
    product = matmul(total, _stage(z, dev))
    return softmax(product, out=out)
