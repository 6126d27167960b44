/*
 * hexmi.h - C ABI of libhexmi.so: hand-written gfx950 (MI355X) kernels for the
 * operator set that hexagon-mlir lowers its tutorial kernels to.
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is
 *     allocated, freed or retained by the library;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls enqueue work and return without synchronising;
 *   - the return value is HEXMI_OK or a negative hexmi_status; nothing throws;
 *   - calls are re-entrant; two calls may run concurrently on different streams
 *     (the one exception, hexmi_block_sum_static, says so);
 *   - a HEXMI_ELAUNCH status describes the launches of that call only: an
 *     error left pending on the calling thread by earlier HIP calls is
 *     discarded on entry, not reported.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the hexagon-mlir source tree).
 */
#ifndef HEXMI_H
#define HEXMI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *hexmi_stream_t; /* hipStream_t */

typedef enum hexmi_status {
  HEXMI_OK = 0,
  HEXMI_EINVAL = -1,  /* null pointer, non-positive size, bad leading dim, misaligned */
  HEXMI_ENOTSUP = -2, /* dtype / shape combination with no kernel */
  HEXMI_ELAUNCH = -3, /* hipLaunchKernel or another HIP call failed */
  HEXMI_ETOOBIG = -4  /* size beyond the fixed capacity of an entry point that allocates nothing */
} hexmi_status;

/* Element types. The values are the reference's raw-tensor data type ids
 * (enum DataType of test/utils/dsp/include/tensor.h:26-38, the table the device
 * harness and backend/utils.py:36-54 share: Half = 1, Float = 2, Int8 = 4).
 * bfloat16 has no id there; it takes a value outside that table (ids 0..10). */
typedef enum hexmi_dtype {
  HEXMI_F16 = 1,
  HEXMI_F32 = 2,
  HEXMI_I8 = 4,
  HEXMI_BF16 = 16
} hexmi_dtype;

/* Library / device ------------------------------------------------------- */

/* "hexmi <major>.<minor> gfx950" */
const char *hexmi_version(void);
/* Text for a status code. */
const char *hexmi_strerror(int status);
/* Number of compute units of the current device (0 if no device). The
 * reference counterpart is the fixed thread count the launcher passes
 * (backend/hexagon_options.py:24 num_threads). */
int hexmi_num_cus(void);

/* Row reductions --------------------------------------------------------- */

/* y[r, :] = softmax(x[r, :]) for r in [0, rows). exp is evaluated in fp32 for
 * every dtype; max-subtracted; masked columns behave as -inf.
 * Stands in for the compiled `softmax_kernel(x_ptr, output_ptr, NUM_ROWS,
 * NUM_COLS, BLOCK_SIZE)` of test/python/triton/test_softmax.py:44-72 and
 * nn.Softmax(dim=1) of test/python/torch-mlir/test_softmax_torch.py:24-31.
 * ld_x / ld_y: elements between consecutive rows (>= cols).
 * dtype: HEXMI_F32, HEXMI_F16 or HEXMI_BF16 (input and output alike).
 * Rows off the 16-byte boundaries (an odd cols, a view) run within a tenth
 * of the aligned rate when the rows of x and y are equally far off them
 * (x - y and (ld_x - ld_y) * element size multiples of 16 bytes: contiguous
 * tensors, equal column slices), at about two thirds of it otherwise. */
int hexmi_softmax(const void *x, void *y, int64_t rows, int64_t cols,
                  int64_t ld_x, int64_t ld_y, int dtype, hexmi_stream_t stream);

/* y = x * rsqrt(mean(x^2) + eps) * weight, fp32 accumulation.
 * Stands in for `rms_norm_fwd_kernel(x_ptr, y_ptr, weights_ptr, BLOCK_SIZE,
 * EPSILON, NUM_COLS, NUM_ROWS)` of test/python/triton/test_rms_norm.py:37-63.
 * x, y: [rows, cols] contiguous; weight: [cols]; all of `dtype`. */
int hexmi_rms_norm(const void *x, const void *weight, void *y, int64_t rows,
                   int64_t cols, float eps, int dtype, hexmi_stream_t stream);

/* y = (x - mean) * rstd * weight + bias with biased variance, fp32
 * accumulation; mean / rstd (fp32 [rows]) are written when non-NULL.
 * Stands in for `layer_norm_fwd_kernel(x_ptr, y_ptr, weights_ptr, biases_ptr,
 * mean_ptr, rstd_ptr, BLOCK_SIZE, EPSILON, NUM_COLS, NUM_ROWS)` of
 * test/python/triton/test_layer_norm.py:42-82 and nn.LayerNorm of
 * test/python/torch-mlir/test_layernorm_torch.py:24-31.
 * weight / bias may be NULL (treated as 1 / 0). */
int hexmi_layer_norm(const void *x, const void *weight, const void *bias,
                     void *y, float *mean, float *rstd, int64_t rows,
                     int64_t cols, float eps, int dtype, hexmi_stream_t stream);

/* The three row operators with the operands a ranked memref carries and the
 * block size the reference kernels are launched with:
 *  - ld_x / ld_y: elements between consecutive rows (>= cols), as the strides
 *    of the reference's MemRefDescriptor (test/utils/dsp/include/common.h:15-21);
 *  - block_cols: the column block of the kernels' sweeps (BLOCK_SIZE of
 *    test_rms_norm.py:37-63 and test_layer_norm.py:42-82, BLOCK_COL_SIZE of
 *    test/python/triton/test_online_softmax.py:31-81). > 0: every block of
 *    block_cols columns (rounded up to whole 16-byte runs, at most 32 KiB) is
 *    reduced by a workgroup of its own and the per-block statistics are merged:
 *    (max, sum) pairs with the online recurrence of test_online_softmax.py:60-71,
 *    sums of squares, (mean, M2) pairs. 0: the library decides; it splits rows
 *    longer than 128 KiB and problems of fewer rows than half the compute units
 *    whose rows are 32 KiB or longer (the reference's own long-row case is
 *    4 x 65536, test_softmax_scf_multithread.py:19-24; its compiler splits such
 *    reductions over its threads, lib/Conversion/LinalgToLLVM/
 *    SplitReduceGenericPass.cpp), everything else runs the single-pass kernels;
 *  - workspace: fp32 scratch for the per-block statistics of the split form.
 *    hexmi_row_workspace returns the bytes (rows, cols, block_cols, dtype)
 *    take, 0 when the single-pass kernels run. workspace may be NULL (single
 *    pass whatever the shape, up to 128 KiB per row at full speed); one that is
 *    smaller than the query's answer is HEXMI_EINVAL. No initialisation, no
 *    state between calls. Rows, leading dims or pointers that are not
 *    16-byte aligned also run the single-pass kernels.
 * Same results as hexmi_softmax / hexmi_rms_norm / hexmi_layer_norm up to the
 * rounding of the merged statistics. */
int64_t hexmi_row_workspace(int64_t rows, int64_t cols, int64_t block_cols,
                            int dtype);
int hexmi_softmax_ws(const void *x, void *y, int64_t rows, int64_t cols,
                     int64_t ld_x, int64_t ld_y, int64_t block_cols, int dtype,
                     void *workspace, int64_t workspace_bytes,
                     hexmi_stream_t stream);
int hexmi_rms_norm_ws(const void *x, const void *weight, void *y, int64_t rows,
                      int64_t cols, int64_t ld_x, int64_t ld_y, float eps,
                      int64_t block_cols, int dtype, void *workspace,
                      int64_t workspace_bytes, hexmi_stream_t stream);
int hexmi_layer_norm_ws(const void *x, const void *weight, const void *bias,
                        void *y, float *mean, float *rstd, int64_t rows,
                        int64_t cols, int64_t ld_x, int64_t ld_y, float eps,
                        int64_t block_cols, int dtype, void *workspace,
                        int64_t workspace_bytes, hexmi_stream_t stream);

/* Dense GEMM ------------------------------------------------------------- */

/* out[n_row, n_col] (fp32) = act[n_row, n_inner] (fp16) * w[n_inner, n_col]
 * (fp16), all row-major contiguous. Same name order and meaning as the
 * runtime routine the compiler calls for hexkl.matmul:
 * `int hexkl_matmul_f16f16_f32(n_row, n_col, n_inner, outM, inAct, inW)`,
 * qcom_hexagon_backend/bin/runtime/include/HexKLAPI.h:17-20 (body
 * bin/runtime/src/HexKLAPI.cpp:15-141), plus the stream. */
int hexmi_matmul_f16f16_f32(int64_t n_row, int64_t n_col, int64_t n_inner,
                            float *out, const void *act, const void *w,
                            hexmi_stream_t stream);

/* C[M,N] = A[M,K] * op(B); fp32 accumulation on MFMA.
 *   trans_b == 0: B is [K,N] row-major with leading dim ldb (the `matmul`
 *     kernel of test/python/triton/test_matmul.py:35-70: strides (K,1),(N,1),(N,1));
 *   trans_b != 0: B is [N,K] row-major (`x @ W.T`,
 *     test/python/torch-mlir/test_hexkl_macro_matmul.py:24-28).
 * in_dtype: HEXMI_F16 or HEXMI_BF16 (A and B). out_dtype: in_dtype or HEXMI_F32
 * (the fp16 x fp16 -> fp32 form of docs/tutorials/triton/matmul_hexkl.md:61-97).
 * Any shape, leading dimension and alignment of the element type is taken.
 * Fastest: K % 64 == 0, operand rows on 16-byte boundaries (lda, ldb
 * multiples of 8, aligned bases), B as [K,N] with N % 8 == 0; an odd N with B
 * as [N,K] costs about a fifth of the rate, K % 8 == 0 up to half, unaligned
 * operand rows about two thirds. Up to 64 rows against B as [N,K] are a
 * stream of the weights (no tiles).
 * in_dtype == out_dtype == HEXMI_F32: fp32 operands multiplied in fp32 (no
 * rounding of the operands): the fp32 matmuls of the reference's torch-mlir
 * graphs (test/python/torch-mlir/test_add_matmul_softmax.py:25-29). K % 32 == 0
 * with 16-byte aligned rows runs on the fp32 matrix cores, other shapes on the
 * vector ALUs. */
int hexmi_gemm(int64_t M, int64_t N, int64_t K, const void *A, int64_t lda,
               const void *B, int64_t ldb, void *C, int64_t ldc, int in_dtype,
               int out_dtype, int trans_b, hexmi_stream_t stream);

/* hexmi_gemm with the additions of a linear layer fused into its epilogue:
 *   C[m,n] = sum_k A[m,k] * op(B)[k,n] + bias[n] + residual[m,n].
 * bias ([N], contiguous) and residual ([M,N], leading dim ldr) are of the
 * OUTPUT dtype, either may be NULL; both join the fp32 sums in registers and
 * the result is rounded to out_dtype once (a separate add kernel rounds twice).
 * residual may alias C (each element is read by the thread that writes it).
 * Everything else as hexmi_gemm, which is this call with bias = residual =
 * NULL. What it replaces on the reference side: the linalg.generic consumers
 * (bias add, residual add) that the fusion pass pulls into the matmul's loop
 * nest (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:
 * 280-283) instead of leaving them as separate kernels behind the HexKL call
 * (lib/Conversion/LinalgToLLVM/MatmulToHexKLPass.cpp:171-190); the GPT-2
 * block of test/python/torch-mlir/test_gpt2_block.py is four such layers.
 * K == 0 with a bias or residual: HEXMI_ENOTSUP. */
int hexmi_gemm_ex(int64_t M, int64_t N, int64_t K, const void *A, int64_t lda,
                  const void *B, int64_t ldb, void *C, int64_t ldc,
                  const void *bias, const void *residual, int64_t ldr,
                  int in_dtype, int out_dtype, int trans_b,
                  hexmi_stream_t stream);

/* out[M,N] = softmax((x[M,K] + y[M,K]) * z[K,N], over each row), one launch:
 * the fused kernel the reference compiles from
 * test/python/torch-mlir/test_add_matmul_softmax.py:19-29 (torch.add ->
 * torch.matmul -> torch.softmax(dim=-1)). All four matrices row-major of one
 * dtype (HEXMI_F32 / HEXMI_F16 / HEXMI_BF16) with leading dims ldx, ldy, ldz,
 * ldo; the sum x + y is rounded to dtype as torch.add does, the scores stay
 * fp32 until the division. A workgroup owns 32 whole rows, so N is limited:
 * N > hexmi_add_matmul_softmax_max_n() (1024) returns HEXMI_ETOOBIG and the
 * caller runs the three kernels (binary add, hexmi_gemm, hexmi_softmax).
 * Any M, K, leading dims and alignment. */
int64_t hexmi_add_matmul_softmax_max_n(void);
int hexmi_add_matmul_softmax(int64_t M, int64_t N, int64_t K, const void *x,
                             int64_t ldx, const void *y, int64_t ldy,
                             const void *z, int64_t ldz, void *out,
                             int64_t ldo, int dtype, hexmi_stream_t stream);

/* Weight-only int8 GEMM (W8A16): C[m,n] = sum_k A[m,k] * (float(W[n,k]) *
 * float(scales[n])), fp32 accumulation, C fp16.
 * A fp16 [M,K]; W int8 [N,K] row-major (symmetric, zero-point 0); scales fp16
 * [N], one per output channel. Results are reproducible bit for bit; the order
 * of a channel's sum over k may depend on where the channel stands in W (for
 * 2 <= M <= 128 the workgroup that owns it sets the k it starts at), so moving a
 * channel can change its outputs in the last place. Any K: multiples of 64
 * are fastest, multiples of 16 cost little up to 128 rows (passes of 128 rows
 * beyond), other K and unaligned bases run a register-staged tile kernel.
 * The reference has no such kernel; this is the
 * fusion of quant.dcast lowering
 * (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:224-230)
 * with the transposed-weight matmul of test_hexkl_macro_matmul.py:24-28. */
int hexmi_gemm_w8a16(int64_t M, int64_t N, int64_t K, const void *A,
                     const int8_t *W, const void *scales, void *C,
                     hexmi_stream_t stream);

/* hexmi_gemm_w8a16 with a caller-owned scratch buffer, for the shapes whose
 * kernels of choice split K over several workgroups and add the fp32 partial
 * tiles up afterwards: 32 < M <= 128 with more than 48 output channels per
 * compute unit (M = 32: more than 96) or with a long K (up to M = 96: K >= 8192
 * and K > 2 N; above: K >= 4608 + 64 per output channel of a compute unit's
 * share), and 128 < M <= 256 with fewer 128 x 128 tiles than a third of the
 * compute units (than half of them when K >= 8192)
 * (the down projection N = 4096, K = 11008 of
 * the model whose up projection is the benchmark shape is one: M = 256 in 40 us
 * where hexmi_gemm_w8a16 takes 75). hexmi_gemm_w8a16_workspace returns the bytes
 * that takes for (M, N, K) on the current device, 0 when hexmi_gemm_w8a16's own
 * kernels are used anyway. workspace may be NULL (then they are used for every
 * shape the query answers with a size); a workspace smaller than the query's
 * answer is HEXMI_EINVAL. It must
 * be 16-byte aligned, needs no initialisation and holds no state between calls;
 * two calls that overlap in time (different streams) need a workspace each.
 * Partial tiles are added in a fixed order: results are reproducible bit for
 * bit, and permuting output channels permutes the columns of C. The workgroup
 * that adds a tile up waits for the others' partial tiles with a bounded number
 * of polls; they have lower workgroup indices, are dispatched before it and
 * wait for nothing themselves, so the bound is a guard and not a path. Should
 * it ever expire, the sum goes ahead with what the area holds and the first
 * 32-bit word of the workspace reads 1 until the next call clears it (a caller
 * that wants the check reads that word after synchronising the stream).
 * The reference's counterpart is the scratch its matmul runtime routine sets up
 * per call (bin/runtime/src/HexKLAPI.cpp:15-68: VTCM for tiles and the
 * accumulator read-back). */
int64_t hexmi_gemm_w8a16_workspace(int64_t M, int64_t N, int64_t K);
int hexmi_gemm_w8a16_ws(int64_t M, int64_t N, int64_t K, const void *A,
                        const int8_t *W, const void *scales, void *C,
                        void *workspace, int64_t workspace_bytes,
                        hexmi_stream_t stream);

/* out[n,k] (fp32) = float(W[n,k]) * float(scales[n]): the dequantisation the
 * fused kernel applies, exposed so indexing and scale selection can be
 * checked bit-exactly. */
int hexmi_dequant_w8(int64_t N, int64_t K, const int8_t *W, const void *scales,
                     float *out, hexmi_stream_t stream);

/* The other forms of quant.dcast, f = (float(q) - zero_point) * scale "per-tensor
 * or per-axis" (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/
 * LinalgToLLVMPass.cpp:224-230 lowers them, lib/Transforms/
 * SeedLayoutConversions.cpp:135-157 carries the per-axis types):
 * zero_points: int8, one per output channel, or NULL for 0; per_tensor != 0:
 * ONE scale (and one zero point) for the whole tensor, read at index 0.
 * hexmi_dequant_w8_ex writes the fp32 values (float(q) - zero_point is an exact
 * integer and the product one fp32 multiply: bit-exact);
 * hexmi_gemm_w8a16_ex is hexmi_gemm_w8a16 on them: the zero point is subtracted
 * from the widened weights (exact in fp16) inside the kernel, the scale
 * multiplies the finished fp32 sum. Up to 128 rows it runs the kernels of
 * hexmi_gemm_w8a16 (5-15 % slower with zero points, equal with a per-tensor
 * scale alone); more rows run in passes of 128. With zero_points NULL and
 * per_tensor 0 both are the symmetric per-channel entry points above. */
int hexmi_dequant_w8_ex(int64_t N, int64_t K, const int8_t *W,
                        const void *scales, const int8_t *zero_points,
                        int per_tensor, float *out, hexmi_stream_t stream);
int hexmi_gemm_w8a16_ex(int64_t M, int64_t N, int64_t K, const void *A,
                        const int8_t *W, const void *scales,
                        const int8_t *zero_points, int per_tensor, void *C,
                        hexmi_stream_t stream);

/* One-time weight pre-pack for the small-M path: the analogue of the
 * reference's compile-time re-layout of constant matmul weights into the
 * matrix unit's own order (RM -> WH block linearisation,
 * qcom_hexagon_backend/lib/Transforms/PreprocessWeightsForHMXPass.cpp:39-117).
 * Wp holds ceil(N/16)*16*K bytes: tiles of 16 channels x 64 k, tile (t, s) at
 * byte ((t * K/64) + s) * 1024; inside a tile lane l = g*16 + r (0 <= l < 64)
 * holds the 16 bytes W[16t + r][64s + 16g .. 64s + 16g + 16); channels past N
 * are zero. K % 64 == 0. A pure permutation of bytes: bit-exact. */
int hexmi_pack_w8(int64_t N, int64_t K, const int8_t *W, int8_t *Wp,
                  hexmi_stream_t stream);

/* hexmi_gemm_w8a16 on weights packed by hexmi_pack_w8: every weight load of a
 * wave is a contiguous KiB already in MFMA fragment order. K % 1024 == 0 and
 * K <= 4096. Meant for M <= 16 (decode batches); larger M runs 16 rows per
 * launch. hexmi_gemm_w8a16's kernels sum in another order: the results agree
 * to one fp16 unit in the last place. */
int hexmi_gemm_w8a16_packed(int64_t M, int64_t N, int64_t K, const void *A,
                            const int8_t *Wp, const void *scales, void *C,
                            hexmi_stream_t stream);

/* Attention -------------------------------------------------------------- */

/* O = softmax(sm_scale * Q K^T [+ causal mask]) V per (z, h), online softmax
 * with fp32 running max / sum, exp2 with sm_scale*log2(e) folded in.
 * Q, K, V, O: [Z, H, S, D] contiguous (strides H*S*D, S*D, D, 1).
 * Stands in for `attention_fwd_kernel(pid1, Q, K, V, sm_scale, Out, H, N_CTX,
 * BLOCK_M, BLOCK_DMODEL, BLOCK_N, STAGE, stride_0..3)` of
 * test/python/triton/test_flash_attention.py:37-168 (STAGE=1 is causal == 0)
 * and tm_tensor.attention (include/hexagon/Dialect/TmTensor/IR/TmTensorOps.td:28-56).
 * in_dtype: HEXMI_F16 / HEXMI_BF16 (MFMA path) or HEXMI_F32.
 * D: 64 and 128 are the kernels' own sizes; other 16-bit heads up to 256 in
 * multiples of 8 run them on zero-padded tiles (above 128 as two halves);
 * anything else a slow row-wise kernel (D <= 256).
 * out_dtype: in_dtype, or HEXMI_F32 with fp16 inputs (the fp16 QKV -> fp32 O
 * form of test/python/mlir/hexkl_attention/input.mlir:1-169). */
int hexmi_flash_attn_fwd(const void *Q, const void *K, const void *V, void *O,
                         int64_t Z, int64_t H, int64_t S, int64_t D,
                         float sm_scale, int causal, int in_dtype,
                         int out_dtype, hexmi_stream_t stream);

/* tm_tensor.attention: O = softmax(sm_scale * Q K^T + mask) V per batch entry,
 * "Equivalent to : softmax(QK^T / sqrt(d_k) + mask) * V"
 * (include/hexagon/Dialect/TmTensor/IR/TmTensorOps.td:28-56; lowering
 * lib/Transforms/LowerTmTensor.cpp:70-235: scale `:120-123`, additive mask
 * `:157-160`, max / sub / exp / sum / div `:164-222`, P V `:225-229`).
 * Q: [batch, seq_q, head_dim]; K, V: [batch, seq_kv, head_dim];
 * mask: [batch, seq_q, seq_kv] of in_dtype, added to the scaled scores, or
 * NULL; O: [batch, seq_q, head_dim]. The reference fixes
 * sm_scale = 1/sqrt(head_dim); here the caller passes it. -inf mask entries
 * remove a key; a row whose keys are all removed yields NaN, as the
 * reference's max / sub / exp / div sequence does.
 * in_dtype / out_dtype as for hexmi_flash_attn_fwd. */
int hexmi_attention(const void *Q, const void *K, const void *V,
                    const void *mask, void *O, int64_t batch, int64_t seq_q,
                    int64_t seq_kv, int64_t head_dim, float sm_scale,
                    int in_dtype, int out_dtype, hexmi_stream_t stream);

/* Element-wise operators, sum reduction, rotary embedding ------------------ */

/* y[i] = f(x[i]), fp32 arithmetic, result rounded to `dtype`.
 * HEXMI_GELU_TANH: 0.5*x*(1 + tanh(0.797885*x + 0.035677*x^3)), the `gelu_kernel`
 *   of test/python/triton/test_gelu.py:43-54 (checked there against
 *   F.gelu(x, approximate="tanh"));
 * HEXMI_SILU: x / (1 + exp(-x)), `silu_kernel` of test/python/triton/test_silu.py:43-52;
 * HEXMI_RSQRT: test/python/triton/test_rsqrt.py:20-24;
 * HEXMI_SIN / HEXMI_COS: test/python/triton/test_math_ops.py:25-38; HEXMI_EXP. */
typedef enum hexmi_unary_op {
  HEXMI_GELU_TANH = 0,
  HEXMI_SILU = 1,
  HEXMI_RSQRT = 2,
  HEXMI_SIN = 3,
  HEXMI_COS = 4,
  HEXMI_EXP = 5
} hexmi_unary_op;
int hexmi_unary(int op, const void *x, void *y, int64_t n, int dtype,
                hexmi_stream_t stream);

/* y[i] = a[i] (+ - * /) b[i]: `add_kernel` of test/python/triton/test_vec_add.py
 * (and test_vec_add_with_scalar.py:32-46, test_vec_add_2d.py), `div_kernel` of
 * test/python/triton/test_vec_div_2d.py:21-55. 2-D contiguous operands are the
 * same call with n = rows*cols. */
typedef enum hexmi_binary_op {
  HEXMI_ADD = 0,
  HEXMI_SUB = 1,
  HEXMI_MUL = 2,
  HEXMI_DIV = 3
} hexmi_binary_op;
int hexmi_binary(int op, const void *a, const void *b, void *y, int64_t n,
                 int dtype, hexmi_stream_t stream);

/* out[p] = sum(x[p*block .. min((p+1)*block, n))) for p < ceil(n/block): the
 * `sum_kernel` of test/python/triton/test_sum.py:30-36 launched on a grid of
 * ceil(n/block) programs with BLOCK_SIZE = block (the test uses one program over
 * 1024*1024 elements). fp32 accumulation in a fixed order; out has `dtype`. */
int hexmi_block_sum(const void *x, void *out, int64_t n, int64_t block,
                    int dtype, hexmi_stream_t stream);

/* hexmi_block_sum with a caller-owned scratch buffer. A program is one
 * workgroup, as it is one Triton program in the reference, so a launch of a
 * few huge programs (test/python/triton/test_sum.py:25-47 sums 2^20 elements
 * in ONE program) would use one compute unit; with a workspace, programs of
 * 65536 elements and more are summed in two passes over the whole chip (fp32
 * partial sums of runs of 4096 elements, then one sum per program), for every
 * dtype. hexmi_block_sum_workspace returns the bytes that takes for (n, block,
 * dtype): 0 when one pass is used anyway (small programs, or several programs
 * whose size is not a multiple of 4096). workspace may be NULL (one pass);
 * a workspace smaller than the query's answer is HEXMI_EINVAL. The workspace
 * holds no state between calls. */
int64_t hexmi_block_sum_workspace(int64_t n, int64_t block, int dtype);
int hexmi_block_sum_ws(const void *x, void *out, int64_t n, int64_t block,
                       int dtype, void *workspace, int64_t workspace_bytes,
                       hexmi_stream_t stream);

/* hexmi_block_sum_ws without the workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc). It has no counterpart in the reference.
 * The partial sums live in a fixed 1 MiB device array of the library (one
 * copy per GPU, held until the process ends), which bounds the input:
 * n <= hexmi_block_sum_static_max_n() = 2^30 elements, HEXMI_ETOOBIG beyond.
 * Same kernels and same results, bit for bit, as hexmi_block_sum_ws with a
 * workspace. The call allocates and frees nothing. Every call on one GPU uses
 * that GPU's one array: two calls that overlap on the same GPU (different
 * streams or threads) race; calls on one stream are ordered and safe. */
int64_t hexmi_block_sum_static_max_n(void);
int hexmi_block_sum_static(const void *x, void *out, int64_t n, int64_t block,
                           int dtype, hexmi_stream_t stream);

/* One-time re-layout of a constant 16-bit weight matrix: dst[c, r] = src[r, c]
 * for src [rows, cols] (leading dim ld_src >= cols), dst [cols, rows] (ld_dst >=
 * rows); fp16 or bf16 alike (bit patterns are moved). What it replaces: the
 * reference transposes constant rank-2 f16 weights once, at compile time,
 * instead of at every run (qcom_hexagon_backend/lib/Transforms/
 * FoldResourceTransposePass.cpp:21-110), and re-lays constant weights out for
 * the matrix unit (lib/Transforms/PreprocessWeightsForHMXPass.cpp:39-117). Here
 * the layout the matrix-core GEMM streams fastest is the K-contiguous one
 * (hexmi_gemm with trans_b != 0), so a weight stored [K,N] is transposed once
 * and multiplied as B^T from then on. Any shape with rows / 64 <= 65535. */
int hexmi_transpose16(int64_t rows, int64_t cols, const void *src,
                      int64_t ld_src, void *dst, int64_t ld_dst,
                      hexmi_stream_t stream);

/* Rotary position embedding of x [batch, seq, heads, feat] (contiguous, feat
 * even): adjacent feature pairs (2i, 2i+1) are rotated by m * theta^(-2i/feat),
 * m the sequence position: `rope_kernel` of test/python/triton/test_rope.py:97-197
 * (angles `compute_thetas` :43-57, even / odd cases :174-184, torch form
 * `rope_reference_pytorch` :60-95). */
int hexmi_rope(const void *x, void *y, int64_t batch, int64_t seq,
               int64_t heads, int64_t feat, double theta, int dtype,
               hexmi_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HEXMI_H */
