"""The reference's tutorial kernels by name and signature.

A reference call site looks like

    softmax_kernel[grid](x, output, NUM_ROWS=..., NUM_COLS=..., BLOCK_SIZE=...,
                         enableMultiThreading=False, ...)

with host tensors that are updated in place. The objects below accept the
same subscript-then-call form, the same positional / keyword parameters and
the same trailing option flags (see options.py), and run the precompiled
gfx950 kernel instead of compiling one. The SPMD grid only said how many
Hexagon threads share the rows; here it is validated (a grid with fewer than
one program is a ValueError, qcom_hexagon_backend/backend/driver.py:67-74)
and otherwise ignored because the HIP launch covers all rows.
"""
import inspect
import math

from . import ops
from .options import split_options


class Kernel:
    """`kernel[grid](*args, **kwargs)` front for one operator."""

    def __init__(self, fn):
        self._fn = fn
        self._sig = inspect.signature(fn)
        self.__name__ = fn.__name__
        self.__doc__ = fn.__doc__

    def __getitem__(self, grid):
        if callable(grid):
            raise TypeError("hexmi kernels take a literal grid tuple")
        g = tuple(grid) if isinstance(grid, (tuple, list)) else (grid,)
        if len(g) == 0 or len(g) > 3 or math.prod(int(v) for v in g) < 1:
            raise ValueError("Must set at least 1 thread in SPMD launch grid. "
                             "To launch singlethreaded, invoke kernel as follows: your_kernel[(1,)](...)")

        def launch(*args, **kwargs):
            kernel_kwargs, _options = split_options(kwargs)
            bound = self._sig.bind(*args, **kernel_kwargs)   # TypeError on unknown / missing names
            bound.apply_defaults()
            return self._fn(*bound.args, **bound.kwargs)

        return launch

    def __call__(self, *a, **k):
        raise RuntimeError("Cannot call a kernel outside of the kernel[grid](...) form")


def _check_2d(name, t, rows, cols):
    if t.numel() != rows * cols:
        raise ValueError("%s: tensor has %d elements, NUM_ROWS*NUM_COLS = %d" % (name, t.numel(), rows * cols))


@Kernel
def softmax_kernel(x_ptr, output_ptr, NUM_ROWS, NUM_COLS, BLOCK_SIZE=None):
    """test/python/triton/test_softmax.py:44-72 (also test_softmax_scf_multithread.py:37-56)."""
    _check_2d("softmax_kernel", x_ptr, NUM_ROWS, NUM_COLS)
    if BLOCK_SIZE is not None and BLOCK_SIZE < NUM_COLS:
        raise ValueError("BLOCK_SIZE must cover NUM_COLS")
    ops.softmax(x_ptr.view(NUM_ROWS, NUM_COLS), out=output_ptr.view(NUM_ROWS, NUM_COLS))


@Kernel
def online_softmax(x_ptr, output_ptr, NUM_ROWS, NUM_COLS, BLOCK_SIZE=None):
    """test/python/triton/test_online_softmax.py:31-81: same result as softmax_kernel."""
    _check_2d("online_softmax", x_ptr, NUM_ROWS, NUM_COLS)
    ops.softmax(x_ptr.view(NUM_ROWS, NUM_COLS), out=output_ptr.view(NUM_ROWS, NUM_COLS))


@Kernel
def rms_norm_fwd_kernel(x_ptr, y_ptr, weights_ptr, BLOCK_SIZE=None, EPSILON=1e-5, NUM_COLS=None, NUM_ROWS=None):
    """test/python/triton/test_rms_norm.py:37-63."""
    _check_2d("rms_norm_fwd_kernel", x_ptr, NUM_ROWS, NUM_COLS)
    ops.rms_norm(x_ptr.view(NUM_ROWS, NUM_COLS), weights_ptr, EPSILON, out=y_ptr.view(NUM_ROWS, NUM_COLS))


@Kernel
def layer_norm_fwd_kernel(x_ptr, y_ptr, weights_ptr, biases_ptr, mean_ptr, rstd_ptr, BLOCK_SIZE=None,
                          EPSILON=1e-5, NUM_COLS=None, NUM_ROWS=None):
    """test/python/triton/test_layer_norm.py:42-82."""
    _check_2d("layer_norm_fwd_kernel", x_ptr, NUM_ROWS, NUM_COLS)
    ops.layer_norm(x_ptr.view(NUM_ROWS, NUM_COLS), weights_ptr, biases_ptr, EPSILON,
                   out=y_ptr.view(NUM_ROWS, NUM_COLS), mean=mean_ptr, rstd=rstd_ptr)


@Kernel
def matmul(A, B, C, N_ROWS, N_COLUMNS, N_INNER):
    """test/python/triton/test_matmul.py:35-70; with a float32 C this is `matmul_hexkl`
    (docs/tutorials/triton/matmul_hexkl.md:61-97)."""
    if tuple(A.shape) != (N_ROWS, N_INNER) or tuple(B.shape) != (N_INNER, N_COLUMNS):
        raise ValueError("matmul: A must be [N_ROWS,N_INNER] and B [N_INNER,N_COLUMNS]")
    ops.matmul(A, B, out=C)


matmul_hexkl = matmul


@Kernel
def attention_fwd_kernel(pid1, Q, K, V, sm_scale, Out, H, N_CTX, BLOCK_M=None, BLOCK_DMODEL=None, BLOCK_N=None,
                         STAGE=1, stride_0=None, stride_1=None, stride_2=None, stride_3=None):
    """test/python/triton/test_flash_attention.py:37-168. STAGE 1 is the full (non-causal) sweep, STAGE 3
    the causal one; the reference launches one (z,h) per call via pid1, here every (z,h) is computed."""
    if Q.dim() != 4 or Q.shape[1] != H or Q.shape[2] != N_CTX:
        raise ValueError("attention_fwd_kernel: Q must be [Z,H,N_CTX,D]")
    if BLOCK_DMODEL is not None and BLOCK_DMODEL != Q.shape[3]:
        raise ValueError("attention_fwd_kernel: BLOCK_DMODEL must equal the head dimension")
    want = (H * N_CTX * Q.shape[3], N_CTX * Q.shape[3], Q.shape[3], 1)
    given = (stride_0, stride_1, stride_2, stride_3)
    if any(g is not None and g != w for g, w in zip(given, want)):
        raise ValueError("attention_fwd_kernel: only the contiguous [Z,H,N_CTX,D] strides %s are supported" % (want,))
    if STAGE not in (1, 3):
        raise ValueError("attention_fwd_kernel: STAGE must be 1 (full) or 3 (causal)")
    ops.flash_attention(Q, K, V, sm_scale, causal=(STAGE == 3), out=Out)
