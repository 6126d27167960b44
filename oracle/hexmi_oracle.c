/*
 * hexmi_oracle.c - TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the algorithms on the hexagon-mlir hot path
 * (softmax, RMSNorm, LayerNorm, dense matmul, int8-dequant matmul, attention),
 * written from the reference's Triton kernels and MLIR lowerings, with double
 * accumulation so it can serve as ground truth for fp32/fp16 GPU kernels.
 * Only tests, the smoke check and the bench's CPU-baseline leg may load it.
 *
 * Pinning (what each function is checked against, in tests/test_oracle.py):
 *   softmax, online_softmax : torch.softmax on CPU at the reference's shapes
 *       (128x128, 4x65536, non-pow2 columns); rows sum to 1; shift invariance;
 *       two-sweep online recurrence == direct form.
 *   rms_norm, layer_norm    : F.rms_norm / F.layer_norm on CPU at 127x513 and
 *       27x8192; closed forms; mean / rstd against x.mean / var(unbiased=False).
 *   matmul                  : torch.matmul in fp64 on CPU; identity / one-hot /
 *       constant-weight closed forms (dense<1.0>, dense<2.0> weights).
 *   dequant_w8, matmul_w8a16: NOT pinned by anything in the reference (it has
 *       no such kernel). Pinned by closed form only: exact int8*fp16 products,
 *       power-of-two scale patterns, one-hot scales, edge weights +-127 / 0.
 *   attention (brute force) : F.scaled_dot_product_attention on CPU (fp32 and
 *       fp64), causal and full; row 0 of a causal result == V[0].
 *   attention_masked        : F.scaled_dot_product_attention(attn_mask=...) on CPU,
 *                             rectangular (Sq != Skv) and -inf masks; reduces to
 *                             `attention` when mask == NULL and Sq == Skv
 *   attention_online        : the recurrence of the reference kernel, checked
 *       against the brute-force form.
 *   unary (gelu_tanh, silu, rsqrt, sin, cos, exp), binary, block_sum, rope :
 *       F.gelu(approximate="tanh") / F.silu / torch.rsqrt / sin / cos on CPU (the
 *       reference tests' own oracles and tolerances); torch.sum; the reference's
 *       rope_reference_pytorch formula re-stated with torch ops in the test and
 *       the closed forms "position 0 is the identity" / "pairs keep their norm".
 *
 * Storage types: fp16 and bf16 travel as uint16_t bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { OR_F32 = 0, OR_F16 = 1, OR_BF16 = 2 };

/* ---- 16-bit float bit conversions (round-to-nearest-even on the way down) */
static float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: renormalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
  if (absx >= 0x477ff000u) /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  if (absx < 0x33000001u) /* <= 2^-25: rounds to zero */
    return (uint16_t)sign;
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_exp;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    half_exp = 0;
  } else {
    shift = 13;
    half_exp = (uint32_t)(e + 15);
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
  /* q holds the implicit bit for normals: adding it into the exponent field is correct on carry */
  uint32_t out = (half_exp ? ((half_exp - 1) << 10) + q : q);
  return (uint16_t)(sign | out);
}

static float bf16_to_f32(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static double load_el(const void *p, int64_t i, int dtype) {
  switch (dtype) {
    case OR_F32: return (double)((const float *)p)[i];
    case OR_F16: return (double)f16_to_f32(((const uint16_t *)p)[i]);
    default: return (double)bf16_to_f32(((const uint16_t *)p)[i]);
  }
}

static void store_el(void *p, int64_t i, int dtype, double v) {
  switch (dtype) {
    case OR_F32: ((float *)p)[i] = (float)v; break;
    case OR_F16: ((uint16_t *)p)[i] = f32_to_f16((float)v); break;
    default: ((uint16_t *)p)[i] = f32_to_bf16((float)v); break;
  }
}

/* exported for the conversion tests */
uint16_t oracle_f32_to_f16(float f) { return f32_to_f16(f); }
float oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }

/* ---- softmax --------------------------------------------------------------
 * test/python/triton/test_softmax.py:58-72: z = x - max(x); num = exp(z);
 * y = num / sum(num), one row per step. Double arithmetic. */
void oracle_softmax(const void *x, void *y, int64_t rows, int64_t cols, int dtype) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t o = r * cols;
    double m = -INFINITY;
    for (int64_t c = 0; c < cols; ++c) {
      double v = load_el(x, o + c, dtype);
      if (v > m) m = v;
    }
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += exp(load_el(x, o + c, dtype) - m);
    for (int64_t c = 0; c < cols; ++c) store_el(y, o + c, dtype, exp(load_el(x, o + c, dtype) - m) / s);
  }
}

/* test/python/triton/test_online_softmax.py:31-81: sweep 1 keeps a running
 * max m and a running sum l rescaled by alpha = exp(m_old - m_new) per block
 * of `block` columns; sweep 2 writes exp(x - m) / l. fp32 in, fp32 out,
 * single-precision arithmetic as the kernel does. */
void oracle_online_softmax_f32(const float *x, float *y, int64_t rows, int64_t cols, int64_t block) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float m_i = -INFINITY, l_i = 0.0f;
    for (int64_t b0 = 0; b0 < cols; b0 += block) {
      int64_t b1 = b0 + block < cols ? b0 + block : cols;
      float m_ij = m_i;
      for (int64_t c = b0; c < b1; ++c) m_ij = xr[c] > m_ij ? xr[c] : m_ij;
      float l_ij = 0.0f;
      for (int64_t c = b0; c < b1; ++c) l_ij += expf(xr[c] - m_ij);
      float alpha = expf(m_i - m_ij);
      l_i = l_i * alpha + l_ij;
      m_i = m_ij;
    }
    for (int64_t c = 0; c < cols; ++c) y[r * cols + c] = expf(xr[c] - m_i) / l_i;
  }
}

/* ---- RMSNorm: test/python/triton/test_rms_norm.py:50-63 -------------------
 * ms = sum(x*x)/C; rms = sqrt(ms + eps); y = (x / rms) * g. weight may be NULL. */
void oracle_rms_norm(const void *x, const void *w, void *y, int64_t rows, int64_t cols, double eps, int dtype) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t o = r * cols;
    double ss = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      double v = load_el(x, o + c, dtype);
      ss += v * v;
    }
    double rms = sqrt(ss / (double)cols + eps);
    for (int64_t c = 0; c < cols; ++c) {
      double g = w ? load_el(w, c, dtype) : 1.0;
      store_el(y, o + c, dtype, (load_el(x, o + c, dtype) / rms) * g);
    }
  }
}

/* ---- LayerNorm: test/python/triton/test_layer_norm.py:60-82 ---------------
 * mean = sum(x)/C; xc = x - mean; var = sum(xc*xc)/C (biased);
 * rstd = 1/sqrt(var + eps); y = xc*rstd*w + b; mean/rstd (fp32) written when non-NULL. */
void oracle_layer_norm(const void *x, const void *w, const void *b, void *y, float *mean_out, float *rstd_out,
                       int64_t rows, int64_t cols, double eps, int dtype) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const int64_t o = r * cols;
    double s = 0.0;
    for (int64_t c = 0; c < cols; ++c) s += load_el(x, o + c, dtype);
    double mean = s / (double)cols;
    double q = 0.0;
    for (int64_t c = 0; c < cols; ++c) {
      double d = load_el(x, o + c, dtype) - mean;
      q += d * d;
    }
    double rstd = 1.0 / sqrt(q / (double)cols + eps);
    if (mean_out) mean_out[r] = (float)mean;
    if (rstd_out) rstd_out[r] = (float)rstd;
    for (int64_t c = 0; c < cols; ++c) {
      double g = w ? load_el(w, c, dtype) : 1.0;
      double bb = b ? load_el(b, c, dtype) : 0.0;
      store_el(y, o + c, dtype, (load_el(x, o + c, dtype) - mean) * rstd * g + bb);
    }
  }
}

/* ---- dense matmul ----------------------------------------------------------
 * C[M,N] = A[M,K] * B, B given as [K,N] (trans_b == 0; strides (N,1) as in
 * test/python/triton/test_matmul.py:44-60) or as [N,K] (trans_b != 0; x @ W.T,
 * test/python/torch-mlir/test_hexkl_macro_matmul.py:24-28). Scalar triple loop
 * like the fixture's check() (test/python/mlir/hexkl_linalg_matmul/wrapper.cpp:47-67)
 * but with a double accumulator. out_dtype may differ from in_dtype. */
void oracle_matmul(const void *A, const void *B, void *C, int64_t M, int64_t N, int64_t K, int in_dtype,
                   int out_dtype, int trans_b) {
  double *bt = (double *)malloc(sizeof(double) * (size_t)N * (size_t)K); /* [N][K] */
  for (int64_t n = 0; n < N; ++n)
    for (int64_t k = 0; k < K; ++k) bt[n * K + k] = load_el(B, trans_b ? n * K + k : k * N + n, in_dtype);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    double *ar = (double *)malloc(sizeof(double) * (size_t)K);
    for (int64_t k = 0; k < K; ++k) ar[k] = load_el(A, m * K + k, in_dtype);
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      const double *br = bt + n * K;
      for (int64_t k = 0; k < K; ++k) acc += ar[k] * br[k];
      store_el(C, m * N + n, out_dtype, acc);
    }
    free(ar);
  }
  free(bt);
}

/* ---- int8 weight dequantisation and W8A16 matmul ---------------------------
 * quant.dcast semantics (lowered by quant::createLowerQuantOps,
 * qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:224-230):
 * f = (float(q) - zero_point) * scale, per-axis scale on the output channel,
 * symmetric (zero_point 0). int8 -> fp32 is exact and the product is ONE fp32
 * multiply, so the result is defined bit-exactly. */
void oracle_dequant_w8(const int8_t *W, const uint16_t *scales_f16, float *out, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n) {
    float s = f16_to_f32(scales_f16[n]);
    for (int64_t k = 0; k < K; ++k) out[n * K + k] = (float)W[n * K + k] * s;
  }
}

/* C[m,n] = sum_k A[m,k] * dequant(W)[n,k]; A fp16, C fp16; double accumulation
 * of the fp32 dequantised weights. */
void oracle_matmul_w8a16(const uint16_t *A, const int8_t *W, const uint16_t *scales_f16, uint16_t *C, int64_t M,
                         int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float s = f16_to_f32(scales_f16[n]);
    for (int64_t m = 0; m < M; ++m) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)f16_to_f32(A[m * K + k]) * (double)((float)W[n * K + k] * s);
      C[m * N + n] = f32_to_f16((float)acc);
    }
  }
}

/* The asymmetric / per-tensor forms of the same dequantisation (quant.dcast: f = (float(q) - zero_point) * scale,
 * "per-tensor or per-axis", qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:224-230,
 * lib/Transforms/SeedLayoutConversions.cpp:135-157). zero_points may be NULL (0); per_tensor != 0 reads scale and
 * zero point at index 0. The difference of two int8 values is an exact fp32 integer, then ONE fp32 multiply. */
void oracle_dequant_w8_ex(const int8_t *W, const uint16_t *scales_f16, const int8_t *zero_points, int per_tensor,
                          float *out, int64_t N, int64_t K) {
  for (int64_t n = 0; n < N; ++n) {
    const int64_t p = per_tensor ? 0 : n;
    float s = f16_to_f32(scales_f16[p]);
    float zp = zero_points ? (float)zero_points[p] : 0.0f;
    for (int64_t k = 0; k < K; ++k) out[n * K + k] = ((float)W[n * K + k] - zp) * s;
  }
}

void oracle_matmul_w8a16_ex(const uint16_t *A, const int8_t *W, const uint16_t *scales_f16, const int8_t *zero_points,
                            int per_tensor, uint16_t *C, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    const int64_t p = per_tensor ? 0 : n;
    float s = f16_to_f32(scales_f16[p]);
    float zp = zero_points ? (float)zero_points[p] : 0.0f;
    for (int64_t m = 0; m < M; ++m) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)f16_to_f32(A[m * K + k]) * (double)(((float)W[n * K + k] - zp) * s);
      C[m * N + n] = f32_to_f16((float)acc);
    }
  }
}

/* ---- attention -------------------------------------------------------------
 * Brute force: O = softmax(scale * Q K^T + mask) V per (z,h), the form
 * tm_tensor.attention lowers to (qcom_hexagon_backend/lib/Transforms/LowerTmTensor.cpp:120-227:
 * scale, optional additive mask, max / sub / exp / sum / div, then P V).
 * causal != 0 masks key j > query i. Q,K,V: [ZH, S, D] of in_dtype. */
void oracle_attention(const void *Q, const void *K, const void *V, void *O, int64_t ZH, int64_t S, int64_t D,
                      double scale, int causal, int in_dtype, int out_dtype) {
#pragma omp parallel for schedule(dynamic, 4) collapse(2)
  for (int64_t zh = 0; zh < ZH; ++zh) {
    for (int64_t i = 0; i < S; ++i) {
      const int64_t base = zh * S * D;
      const int64_t jend = causal ? i + 1 : S;
      double *p = (double *)malloc(sizeof(double) * (size_t)jend);
      double *acc = (double *)calloc((size_t)D, sizeof(double));
      double m = -INFINITY;
      for (int64_t j = 0; j < jend; ++j) {
        double s = 0.0;
        for (int64_t d = 0; d < D; ++d)
          s += load_el(Q, base + i * D + d, in_dtype) * load_el(K, base + j * D + d, in_dtype);
        p[j] = s * scale;
        if (p[j] > m) m = p[j];
      }
      double l = 0.0;
      for (int64_t j = 0; j < jend; ++j) {
        p[j] = exp(p[j] - m);
        l += p[j];
      }
      for (int64_t j = 0; j < jend; ++j)
        for (int64_t d = 0; d < D; ++d) acc[d] += p[j] * load_el(V, base + j * D + d, in_dtype);
      for (int64_t d = 0; d < D; ++d) store_el(O, base + i * D + d, out_dtype, acc[d] / l);
      free(p);
      free(acc);
    }
  }
}

/* tm_tensor.attention with its mask operand and separate query / key lengths
 * (qcom_hexagon_backend/lib/Transforms/LowerTmTensor.cpp:88-99 shapes, :120-123 scale, :157-160 additive mask,
 * :164-222 softmax, :225-229 P V). Q: [B, Sq, D]; K, V: [B, Skv, D]; mask: [B, Sq, Skv] of in_dtype or NULL. */
void oracle_attention_masked(const void *Q, const void *K, const void *V, const void *mask, void *O, int64_t B,
                             int64_t Sq, int64_t Skv, int64_t D, double scale, int in_dtype, int out_dtype) {
#pragma omp parallel for schedule(dynamic, 4) collapse(2)
  for (int64_t b = 0; b < B; ++b) {
    for (int64_t i = 0; i < Sq; ++i) {
      const int64_t qb = b * Sq * D, kb = b * Skv * D, mb = (b * Sq + i) * Skv;
      double *p = (double *)malloc(sizeof(double) * (size_t)Skv);
      double *acc = (double *)calloc((size_t)D, sizeof(double));
      double m = -INFINITY;
      for (int64_t j = 0; j < Skv; ++j) {
        double s = 0.0;
        for (int64_t d = 0; d < D; ++d)
          s += load_el(Q, qb + i * D + d, in_dtype) * load_el(K, kb + j * D + d, in_dtype);
        p[j] = s * scale + (mask ? load_el(mask, mb + j, in_dtype) : 0.0);
        if (p[j] > m) m = p[j];
      }
      double l = 0.0;
      for (int64_t j = 0; j < Skv; ++j) {
        p[j] = exp(p[j] - m);                  /* m == -inf (every key removed): exp(nan), as the reference */
        l += p[j];
      }
      for (int64_t j = 0; j < Skv; ++j)
        for (int64_t d = 0; d < D; ++d) acc[d] += p[j] * load_el(V, kb + j * D + d, in_dtype);
      for (int64_t d = 0; d < D; ++d) store_el(O, qb + i * D + d, out_dtype, acc[d] / l);
      free(p);
      free(acc);
    }
  }
}

/* The reference kernel's recurrence (test/python/triton/test_flash_attention.py:54-77,144-168):
 * m_i = -99999999999999.0, l_i = 1.0, acc = 0; qk_scale = sm_scale * 1.44269504;
 * per block of block_n keys: m_ij = max(m_i, max(qk)*qk_scale); p = exp2(qk*qk_scale - m_ij);
 * alpha = exp2(m_i - m_ij); l_i = l_i*alpha + sum(p); acc = acc*alpha + p V; out = acc / l_i.
 * fp32 in / out, single-precision arithmetic; STAGE 1 only (no mask), as the reference runs it. */
void oracle_attention_online_f32(const float *Q, const float *K, const float *V, float *O, int64_t ZH, int64_t S,
                                 int64_t D, float sm_scale, int64_t block_n) {
  const float qk_scale = sm_scale * 1.44269504f;
  float *acc = (float *)malloc(sizeof(float) * (size_t)D);
  float *qk = (float *)malloc(sizeof(float) * (size_t)block_n);
  for (int64_t zh = 0; zh < ZH; ++zh) {
    const float *q = Q + zh * S * D, *k = K + zh * S * D, *v = V + zh * S * D;
    for (int64_t i = 0; i < S; ++i) {
      float m_i = -99999999999999.0f, l_i = 1.0f;
      for (int64_t d = 0; d < D; ++d) acc[d] = 0.0f;
      for (int64_t j0 = 0; j0 < S; j0 += block_n) {
        int64_t nb = j0 + block_n < S ? block_n : S - j0;
        float mx = -INFINITY;
        for (int64_t j = 0; j < nb; ++j) {
          float s = 0.0f;
          for (int64_t d = 0; d < D; ++d) s += q[i * D + d] * k[(j0 + j) * D + d];
          qk[j] = s;
          if (s > mx) mx = s;
        }
        float m_ij = fmaxf(m_i, mx * qk_scale);
        float l_ij = 0.0f;
        for (int64_t j = 0; j < nb; ++j) {
          qk[j] = exp2f(qk[j] * qk_scale - m_ij);
          l_ij += qk[j];
        }
        float alpha = exp2f(m_i - m_ij);
        l_i = l_i * alpha + l_ij;
        for (int64_t d = 0; d < D; ++d) {
          float a = acc[d] * alpha;
          for (int64_t j = 0; j < nb; ++j) a += qk[j] * v[(j0 + j) * D + d];
          acc[d] = a;
        }
        m_i = m_ij;
      }
      for (int64_t d = 0; d < D; ++d) O[zh * S * D + i * D + d] = acc[d] / l_i;
    }
  }
  free(acc);
  free(qk);
}

/* ---- element-wise operators, block sums, rotary embedding -------------------
 * op codes as hexmi_unary_op / hexmi_binary_op. */
void oracle_unary(int op, const void *x, void *y, int64_t n, int dtype) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    const double v = load_el(x, i, dtype);
    double r;
    switch (op) {
      case 0: { /* gelu_kernel, test/python/triton/test_gelu.py:26-30,54 (its own constants) */
        const double u = 0.797885 * v + 0.035677 * v * v * v;
        r = 0.5 * v * (1.0 + tanh(u));
        break;
      }
      case 1: r = v / (1.0 + exp(-v)); break;            /* test_silu.py:50 */
      case 2: r = 1.0 / sqrt(v); break;                  /* test_rsqrt.py:20-24 */
      case 3: r = sin(v); break;                         /* test_math_ops.py:33-38 */
      case 4: r = cos(v); break;                         /* test_math_ops.py:25-30 */
      default: r = exp(v); break;
    }
    store_el(y, i, dtype, r);
  }
}

void oracle_binary(int op, const void *a, const void *b, void *y, int64_t n, int dtype) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    const double u = load_el(a, i, dtype), v = load_el(b, i, dtype);
    store_el(y, i, dtype, op == 0 ? u + v : op == 1 ? u - v : op == 2 ? u * v : u / v);
  }
}

/* sum_kernel, test/python/triton/test_sum.py:30-36: out[pid] = sum of program pid's BLOCK_SIZE elements */
void oracle_block_sum(const void *x, void *out, int64_t n, int64_t block, int dtype) {
  const int64_t programs = (n + block - 1) / block;
  for (int64_t p = 0; p < programs; ++p) {
    const int64_t end = (p + 1) * block < n ? (p + 1) * block : n;
    double s = 0.0;
    for (int64_t i = p * block; i < end; ++i) s += load_el(x, i, dtype);
    store_el(out, p, dtype, s);
  }
}

/* rope_kernel, test/python/triton/test_rope.py:43-57 (angles), :174-184 (even / odd cases):
 * x [batch, seq, heads, feat]; pair (2i, 2i+1) at position m turns by m / theta^(2i/feat). */
void oracle_rope(const void *x, void *y, int64_t batch, int64_t seq, int64_t heads, int64_t feat, double theta,
                 int dtype) {
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t m = 0; m < seq; ++m)
      for (int64_t h = 0; h < heads; ++h)
        for (int64_t i = 0; i < feat; i += 2) {
          const int64_t off = ((b * seq + m) * heads + h) * feat + i;
          const double ang = (double)m / pow(theta, (double)i / (double)feat);
          const double e = load_el(x, off, dtype), o = load_el(x, off + 1, dtype);
          store_el(y, off, dtype, e * cos(ang) - o * sin(ang));
          store_el(y, off + 1, dtype, e * sin(ang) + o * cos(ang));
        }
}
