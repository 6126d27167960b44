"""hexmi: MI355X (gfx950) kernels behind the operator API of hexagon-mlir's tutorial kernels."""
from ._lib import HexmiError, LIB_PATH, lib  # noqa: F401
from .ops import (add_matmul_softmax, attention, binary, block_sum, dequant_w8, flash_attention, gelu, pack_w8, pack_weight, rope, silu, unary,
                  w8a16_matmul_packed, layer_norm, matmul, rms_norm, softmax,  # noqa: F401
                  w8a16_matmul, through_dispatcher)
from . import kernels  # noqa: F401
from .tensor_file import load_tensor, save_tensor  # noqa: F401

__all__ = ["load_tensor", "save_tensor", "softmax", "rms_norm", "layer_norm", "matmul", "w8a16_matmul", "dequant_w8", "pack_w8", "pack_weight", "w8a16_matmul_packed", "flash_attention", "attention", "add_matmul_softmax", "unary", "binary", "gelu", "silu", "block_sum", "rope",
           "kernels", "HexmiError", "lib", "LIB_PATH", "through_dispatcher"]
