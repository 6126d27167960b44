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
def online_softmax(x_ptr, output_ptr, NUM_ROWS, NUM_COLS, BLOCK_ROW_SIZE=None, BLOCK_COL_SIZE=None):
    """test/python/triton/test_online_softmax.py:31-81: the two-phase softmax over column blocks of BLOCK_COL_SIZE
    (running max and sum per row, then the normalising sweep). Here every column block of a row is reduced by a
    workgroup of its own and the (max, sum) pairs are merged with the same recurrence; BLOCK_ROW_SIZE, the rows of a
    program, has no counterpart (the grid covers all rows)."""
    _check_2d("online_softmax", x_ptr, NUM_ROWS, NUM_COLS)
    block = int(BLOCK_COL_SIZE) if BLOCK_COL_SIZE else NUM_COLS
    if block <= 0 or NUM_COLS % block != 0:
        raise ValueError("BLOCK_COL_SIZE must divide NUM_COLS")
    ops.softmax(x_ptr.view(NUM_ROWS, NUM_COLS), out=output_ptr.view(NUM_ROWS, NUM_COLS), block_cols=block)


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
    the causal one. pid1 selects the (z, h) pair the launch works on, as in the reference (off_hz = pid1,
    off_z = pid1 // H, off_h = pid1 % H, `:102-105`; its test passes 0 with Z = H = 1): a caller that loops pid1
    over Z * H gets each head computed once. pid1=None (no counterpart in the reference) computes every head in
    one launch."""
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
    if pid1 is None:
        ops.flash_attention(Q, K, V, sm_scale, causal=(STAGE == 3), out=Out)
        return
    pid1 = int(pid1)
    if not 0 <= pid1 < Q.shape[0] * H:
        raise ValueError("attention_fwd_kernel: pid1 must be in [0, Z*H)")
    z, h = pid1 // H, pid1 % H
    ops.flash_attention(Q[z:z + 1, h:h + 1], K[z:z + 1, h:h + 1], V[z:z + 1, h:h + 1], sm_scale, causal=(STAGE == 3),
                        out=Out[z:z + 1, h:h + 1])


def _check_block(name, t, BLOCK_SIZE, programs):
    if BLOCK_SIZE is not None and BLOCK_SIZE * programs < t.numel():
        raise ValueError("%s: grid of %d programs x BLOCK_SIZE %d does not cover %d elements"
                         % (name, programs, BLOCK_SIZE, t.numel()))


@Kernel
def gelu_kernel(x_ptr, output_ptr, BLOCK_SIZE=None):
    """test/python/triton/test_gelu.py:43-54."""
    ops.unary("gelu_tanh", x_ptr, out=output_ptr)


@Kernel
def silu_kernel(x_ptr, output_ptr, BLOCK_SIZE=None):
    """test/python/triton/test_silu.py:43-52."""
    ops.unary("silu", x_ptr, out=output_ptr)


@Kernel
def rsqrt_kernel(x_ptr, output_ptr, BLOCK_SIZE=None):
    """test/python/triton/test_rsqrt.py:20-24."""
    ops.unary("rsqrt", x_ptr, out=output_ptr)


@Kernel
def sin_kernel(x_ptr, output_ptr, BLOCK_SIZE=None):
    """test/python/triton/test_math_ops.py:33-38."""
    ops.unary("sin", x_ptr, out=output_ptr)


@Kernel
def cos_kernel(x_ptr, output_ptr, BLOCK_SIZE=None):
    """test/python/triton/test_math_ops.py:25-30."""
    ops.unary("cos", x_ptr, out=output_ptr)


@Kernel
def add_kernel(x_ptr, y_ptr, output_ptr, n_elements=None, BLOCK_SIZE=None):
    """test/python/triton/test_vec_add.py (and test_vec_add_with_scalar.py:32-46: n_elements masks the tail)."""
    if n_elements is not None and n_elements != x_ptr.numel():
        ops.binary("add", x_ptr.reshape(-1)[:n_elements], y_ptr.reshape(-1)[:n_elements],
                   out=output_ptr.reshape(-1)[:n_elements])
    else:
        ops.binary("add", x_ptr, y_ptr, out=output_ptr)


add_kernel_scalar = add_kernel


@Kernel
def div_kernel(x_ptr, y_ptr, output_ptr, NUM_ROWS=None, NUM_COLS=None):
    """test/python/triton/test_vec_div_2d.py:21-55."""
    if NUM_ROWS is not None and NUM_COLS is not None:
        _check_2d("div_kernel", x_ptr, NUM_ROWS, NUM_COLS)
    ops.binary("div", x_ptr, y_ptr, out=output_ptr)


class _SumKernel(Kernel):
    """`sum_kernel[grid](x, out, BLOCK_SIZE=...)` writes one sum per program, so the launch needs the grid."""

    def __getitem__(self, grid):
        launch = super().__getitem__(grid)
        g = tuple(grid) if isinstance(grid, (tuple, list)) else (grid,)
        programs = math.prod(int(v) for v in g)

        def with_grid(*args, **kwargs):
            return launch(*args, _programs=programs, **kwargs)

        return with_grid


@_SumKernel
def sum_kernel(x_ptr, output_ptr, BLOCK_SIZE=None, _programs=1):
    """test/python/triton/test_sum.py:30-36: program p stores the sum of elements [p*BLOCK_SIZE, (p+1)*BLOCK_SIZE)."""
    if BLOCK_SIZE is None:
        BLOCK_SIZE = x_ptr.numel()
    _check_block("sum_kernel", x_ptr, BLOCK_SIZE, _programs)
    if output_ptr.numel() < _programs:
        raise ValueError("sum_kernel: output must hold one element per program")
    n = min(x_ptr.numel(), BLOCK_SIZE * _programs)
    used = (n + BLOCK_SIZE - 1) // BLOCK_SIZE
    ops.block_sum(x_ptr.reshape(-1)[:n], BLOCK_SIZE, out=output_ptr.reshape(-1)[:used])


@Kernel
def rope_kernel(x_ptr, output_ptr, BATCH_SIZE, BATCH_SIZE_STRIDE, SEQ_LEN, SEQ_LEN_STRIDE, N_HEADS, N_HEADS_STRIDE,
                N_FEATURES, N_FEATURES_STRIDE, BLOCK_SIZE=None, THETA=10000.0):
    """test/python/triton/test_rope.py:97-197; only the contiguous [B, L, H, F] strides are supported."""
    want = (SEQ_LEN * N_HEADS * N_FEATURES, N_HEADS * N_FEATURES, N_FEATURES, 1)
    if (BATCH_SIZE_STRIDE, SEQ_LEN_STRIDE, N_HEADS_STRIDE, N_FEATURES_STRIDE) != want:
        raise ValueError("rope_kernel: only the contiguous strides %s are supported" % (want,))
    if x_ptr.numel() != BATCH_SIZE * want[0]:
        raise ValueError("rope_kernel: tensor does not have BATCH_SIZE*SEQ_LEN*N_HEADS*N_FEATURES elements")
    shape = (BATCH_SIZE, SEQ_LEN, N_HEADS, N_FEATURES)
    ops.rope(x_ptr.view(shape), THETA, out=output_ptr.view(shape))
