// out = softmax((x + y) z) over each row, in one launch: the graph of
// test/python/torch-mlir/test_add_matmul_softmax.py:19-29 (torch.add -> torch.matmul -> torch.softmax(dim=-1)), which
// the reference's fusion pass (qcom_hexagon_backend/lib/Conversion/LinalgToLLVM/LinalgToLLVMPass.cpp:280-283) turns
// into one kernel. Here: a workgroup owns 32 whole rows of the result (N <= 1024 columns), so the softmax is an
// epilogue of the product and neither the sum x + y nor the product is ever written to memory.
//
//  - prologue: the A operand is staged as T(x + y) (the rounding torch.add gives the sum), 16 elements of K a step;
//  - product on the matrix cores: v_mfma_f32_32x32x16 for fp16 / bf16, v_mfma_f32_32x32x2_f32 for fp32 (no
//    rounding of fp32 operands), z staged [n][k]; wave w owns columns [w * 32 * NT, (w + 1) * 32 * NT);
//  - epilogue: the MFMA is issued with z as its first operand, so a lane holds 16 * NT columns of ONE row
//    (row lane % 32): the row maximum and sum are thread-local loops, one exchange with lane ^ 32 and one pass
//    through LDS across the four waves. The scores stay fp32 from the product to the division.
//
// Any M, K, leading dimensions and alignment (guarded scalar copies); N > 1024 is not taken (the caller runs the
// three kernels). The kernel re-reads z once per 32 rows, so it is the choice for small and skinny problems; large
// products are faster as add -> tiled GEMM -> softmax.
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr int kRows = 32;     // rows of the result per workgroup
constexpr int kStepK = 16;    // elements of K staged per step
constexpr int kMaxN = 1024;   // 4 waves x 8 tiles x 32 columns

template <typename T> struct StepMma;
template <> struct StepMma<f16> {
  static constexpr int PAD = 8;
  // acc[r] += sum_k b_row[k] * a_row[k]: result "row" index = column of z (lane % 32 of b), "column" = row of x
  static __device__ __forceinline__ f32x16 run(const f16* b_row, const f16* a_row, int half, f32x16 acc) {
    const f16x8 bf = *reinterpret_cast<const f16x8*>(b_row + half * 8);
    const f16x8 af = *reinterpret_cast<const f16x8*>(a_row + half * 8);
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(bf, af, acc, 0, 0, 0);
  }
};
template <> struct StepMma<bf16> {
  static constexpr int PAD = 8;
  static __device__ __forceinline__ f32x16 run(const bf16* b_row, const bf16* a_row, int half, f32x16 acc) {
    const bf16x8 bf = *reinterpret_cast<const bf16x8*>(b_row + half * 8);
    const bf16x8 af = *reinterpret_cast<const bf16x8*>(a_row + half * 8);
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf, af, acc, 0, 0, 0);
  }
};
template <> struct StepMma<float> {
  static constexpr int PAD = 4;
  static __device__ __forceinline__ f32x16 run(const float* b_row, const float* a_row, int half, f32x16 acc) {
#pragma unroll
    for (int e = 0; e < kStepK / 2; ++e)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b_row[2 * e + half], a_row[2 * e + half], acc, 0, 0, 0);
    return acc;
  }
};

// NT: 32-column tiles per wave; the workgroup covers 128 * NT columns.
template <typename T, int NT>
__global__ __launch_bounds__(256)
void add_matmul_softmax_kernel(const T* __restrict__ x, const T* __restrict__ y, const T* __restrict__ z,
                               T* __restrict__ out, int M, int N, int K, int64_t ldx, int64_t ldy, int64_t ldz,
                               int64_t ldo, bool runs) {
  constexpr int PITCH = kStepK + StepMma<T>::PAD;
  constexpr int COLS = 128 * NT;
  __shared__ __attribute__((aligned(16))) T a_s[kRows * PITCH];    // [row][k]: T(x + y)
  __shared__ __attribute__((aligned(16))) T b_s[COLS * PITCH];     // [column][k]: z
  __shared__ float red[4][kRows];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int half = lane / 32, lrow = lane % 32;
  const int m0 = blockIdx.x * kRows;
  f32x16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += kStepK) {
    __syncthreads();
    for (int e = threadIdx.x; e < kRows * kStepK; e += 256) {
      const int r = e / kStepK, k = e % kStepK;
      const int gm = m0 + r, gk = k0 + k;
      float v = 0.0f;
      if (gm < M && gk < K) v = to_f32<T>(x[(int64_t)gm * ldx + gk]) + to_f32<T>(y[(int64_t)gm * ldy + gk]);
      a_s[r * PITCH + k] = from_f32<T>(v);
    }
    for (int e = threadIdx.x; e < COLS * kStepK; e += 256) {
      const int n = e % COLS, k = e / COLS;         // consecutive threads read consecutive columns of one row of z
      const int gk = k0 + k;
      b_s[n * PITCH + k] = (n < N && gk < K) ? z[(int64_t)gk * ldz + n] : from_f32<T>(0.0f);
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NT; ++t)
      acc[t] = StepMma<T>::run(b_s + ((wave * NT + t) * 32 + lrow) * PITCH, a_s + lrow * PITCH, half, acc[t]);
  }

  // acc[t][r]: row m0 + lane % 32, column (wave * NT + t) * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4
  const int cbase = wave * NT * 32 + 4 * half;
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int col = cbase + t * 32 + 8 * (r / 4) + r % 4;
      if (col >= N) acc[t][r] = -INFINITY;
      mx = fmaxf(mx, acc[t][r]);
    }
  mx = fmaxf(mx, __shfl_xor(mx, 32));
  if (half == 0) red[wave][lrow] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0][lrow], red[1][lrow]), fmaxf(red[2][lrow], red[3][lrow]));   // finite: column 0 exists
  __syncthreads();
  float sum = 0.0f;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc[t][r] = __expf(acc[t][r] - mx);
      sum += acc[t][r];
    }
  sum += __shfl_xor(sum, 32);
  if (half == 0) red[wave][lrow] = sum;
  __syncthreads();
  const float inv = 1.0f / (red[0][lrow] + red[1][lrow] + red[2][lrow] + red[3][lrow]);

  const int row = m0 + lrow;
  if (row >= M) return;
  T* orow = out + (int64_t)row * ldo;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int col = cbase + t * 32 + 8 * q;
      if (runs && col + 3 < N) {
        store4<T>(orow + col, acc[t][4 * q] * inv, acc[t][4 * q + 1] * inv, acc[t][4 * q + 2] * inv,
                  acc[t][4 * q + 3] * inv);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (col + r < N) orow[col + r] = from_f32<T>(acc[t][4 * q + r] * inv);
      }
    }
}

template <typename T>
int launch(const void* x, const void* y, const void* z, void* out, int64_t M, int64_t N, int64_t K, int64_t ldx,
           int64_t ldy, int64_t ldz, int64_t ldo, hipStream_t s) {
  const dim3 grid((unsigned)((M + kRows - 1) / kRows));
  const bool runs = ldo % 4 == 0 && aligned_to(out, 4 * sizeof(T));   // results leave in runs of four columns
#define HEXMI_LAUNCH(NT)                                                                                            \
  hipLaunchKernelGGL((add_matmul_softmax_kernel<T, NT>), grid, dim3(256), 0, s, static_cast<const T*>(x),           \
                     static_cast<const T*>(y), static_cast<const T*>(z), static_cast<T*>(out), (int)M, (int)N, (int)K, \
                     ldx, ldy, ldz, ldo, runs)
  if (N <= 128) HEXMI_LAUNCH(1);
  else if (N <= 256) HEXMI_LAUNCH(2);
  else if (N <= 512) HEXMI_LAUNCH(4);
  else HEXMI_LAUNCH(8);
#undef HEXMI_LAUNCH
  return launch_status();
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" int64_t hexmi_add_matmul_softmax_max_n(void) { return kMaxN; }

extern "C" int hexmi_add_matmul_softmax(int64_t M, int64_t N, int64_t K, const void* x, int64_t ldx, const void* y,
                                        int64_t ldy, const void* z, int64_t ldz, void* out, int64_t ldo, int dtype,
                                        hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!out || (K > 0 && (!x || !y || !z))) return HEXMI_EINVAL;
  if (ldx < K || ldy < K || ldz < N || ldo < N) return HEXMI_EINVAL;
  if (N > kMaxN) return HEXMI_ETOOBIG;
  if (M > 0x7fffffff - kRows || K > 0x7fffffff - kStepK) return HEXMI_ENOTSUP;
  begin_call();
  hipStream_t s = as_stream(stream);
  // K == 0: every score is the empty sum 0, every row the uniform distribution; the kernel's loop does not run
  switch (dtype) {
    case HEXMI_F32: return launch<float>(x, y, z, out, M, N, K, ldx, ldy, ldz, ldo, s);
    case HEXMI_F16: return launch<f16>(x, y, z, out, M, N, K, ldx, ldy, ldz, ldo, s);
    case HEXMI_BF16: return launch<bf16>(x, y, z, out, M, N, K, ldx, ldy, ldz, ldo, s);
    default: return HEXMI_ENOTSUP;
  }
}
