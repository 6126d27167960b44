"""ctypes loader for libhexmi.so (the C ABI declared in include/hexmi.h).

There is no fallback: if the library has not been built the import of any
operator raises, and every non-zero status from the library raises
HexmiError.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhexmi.so")

OK, EINVAL, ENOTSUP, ELAUNCH, ETOOBIG = 0, -1, -2, -3, -4
F16, F32, I8, BF16 = 1, 2, 4, 16       # hexmi_dtype: the reference's tensor.h ids, bf16 outside its table


class HexmiError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__("%s failed with status %d: %s" % (what, status, strerror(status)))


_c = ctypes
_i64, _int, _f32, _f64, _ptr = _c.c_int64, _c.c_int, _c.c_float, _c.c_double, _c.c_void_p

# name -> (restype, argtypes); must list every symbol of include/hexmi.h (the operator ABI)
SIGNATURES = {
    "hexmi_version": (_c.c_char_p, []),
    "hexmi_strerror": (_c.c_char_p, [_int]),
    "hexmi_num_cus": (_int, []),
    "hexmi_softmax": (_int, [_ptr, _ptr, _i64, _i64, _i64, _i64, _int, _ptr]),
    "hexmi_rms_norm": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _f32, _int, _ptr]),
    "hexmi_layer_norm": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _int, _ptr]),
    "hexmi_row_workspace": (_i64, [_i64, _i64, _i64, _int]),
    "hexmi_softmax_ws": (_int, [_ptr, _ptr, _i64, _i64, _i64, _i64, _i64, _int, _ptr, _i64, _ptr]),
    "hexmi_rms_norm_ws": (_int, [_ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _f32, _i64, _int, _ptr, _i64, _ptr]),
    "hexmi_layer_norm_ws": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _f32, _i64, _int, _ptr,
                                   _i64, _ptr]),
    "hexmi_matmul_f16f16_f32": (_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "hexmi_gemm": (_int, [_i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _int, _int, _int, _ptr]),
    "hexmi_gemm_ex": (_int, [_i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _i64, _int, _int, _int,
                             _ptr]),
    "hexmi_add_matmul_softmax_max_n": (_i64, []),
    "hexmi_add_matmul_softmax": (_int, [_i64, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _int, _ptr]),
    "hexmi_transpose16": (_int, [_i64, _i64, _ptr, _i64, _ptr, _i64, _ptr]),
    "hexmi_gemm_w8a16": (_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "hexmi_gemm_w8a16_workspace": (_i64, [_i64, _i64, _i64]),
    "hexmi_gemm_w8a16_ws": (_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "hexmi_pack_w8": (_int, [_i64, _i64, _ptr, _ptr, _ptr]),
    "hexmi_gemm_w8a16_packed": (_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "hexmi_dequant_w8": (_int, [_i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "hexmi_dequant_w8_ex": (_int, [_i64, _i64, _ptr, _ptr, _ptr, _int, _ptr, _ptr]),
    "hexmi_gemm_w8a16_ex": (_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _int, _ptr, _ptr]),
    "hexmi_flash_attn_fwd": (_int, [_ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _f32, _int, _int, _int, _ptr]),
    "hexmi_unary": (_int, [_int, _ptr, _ptr, _i64, _int, _ptr]),
    "hexmi_binary": (_int, [_int, _ptr, _ptr, _ptr, _i64, _int, _ptr]),
    "hexmi_block_sum": (_int, [_ptr, _ptr, _i64, _i64, _int, _ptr]),
    "hexmi_block_sum_workspace": (_i64, [_i64, _i64, _int]),
    "hexmi_block_sum_ws": (_int, [_ptr, _ptr, _i64, _i64, _int, _ptr, _i64, _ptr]),
    "hexmi_block_sum_static_max_n": (_i64, []),
    "hexmi_block_sum_static": (_int, [_ptr, _ptr, _i64, _i64, _int, _ptr]),
    "hexmi_rope": (_int, [_ptr, _ptr, _i64, _i64, _i64, _i64, _f64, _int, _ptr]),
    "hexmi_attention": (_int, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _f32, _int, _int, _ptr]),
}

# measurement probes of include/hexmi_calibrate.h: exported by the library, not part of the operator ABI
PROBE_SIGNATURES = {
    "hexmi_mfma_peak_flops": (_f64, [_int, _int, _i64]),
    "hexmi_mfma_peak": (_int, [_int, _int, _ptr, _i64, _int, _ptr, _ptr]),
    "hexmi_issue_slots": (_int, [_int, _int, _int, _i64, _int, _ptr, _ptr]),
    "hexmi_lds_read_pattern": (_int, [_int, _i64, _ptr, _ptr]),
    "hexmi_l2_stream": (_int, [_int, _int, _i64, _i64, _ptr, _ptr, _ptr]),
}

_lib = None


def lib():
    """The loaded library; raises if it was never built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libhexmi.so is missing at %s: build it with `python hexagon-mlir_amd/build.py` "
                "(there is no CPU or eager fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in list(SIGNATURES.items()) + list(PROBE_SIGNATURES.items()):
            fn = getattr(handle, name)          # AttributeError if the symbol is not exported
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def strerror(status):
    return lib().hexmi_strerror(int(status)).decode()


def check(status, what):
    if status != OK:
        raise HexmiError(status, what)
