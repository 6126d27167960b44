// Weight-only int8 GEMM (W8A16): C[m,n] = scale[n] * sum_k A[m,k] * W[n,k], fp16 activations, int8 weights,
// fp32 accumulation on 16x16x32 matrix-core tiles, fp16 output.
//
// The weight matrix is the only large operand (N*K bytes) and every weight is used once per 16 activation rows,
// so weights never touch LDS: each lane fetches 16 consecutive int8 of one output channel straight from HBM
// (16-byte loads, a 16-channel tile reads 64 contiguous bytes per channel per instruction), converts them to
// fp16 in registers and feeds two MFMAs. int8 -> fp16 is exact: byte b = w ^ 0x80 placed in the low mantissa
// bits of 0x6400 is the fp16 number 1024 + b, and subtracting 1152 leaves w.
//
// The per-channel scale multiplies the finished fp32 sum (it is constant over k), which differs from
// "dequantise, then multiply" only by fp32 rounding; hexmi_dequant_w8 exposes the element-wise dequantisation.
//
// Work split: a workgroup of 8 waves owns one tile of 16 output channels at a time; the waves split K eight ways
// and their partial tiles are summed through LDS. Activations are staged in LDS once per workgroup when they
// fit (16*MT rows x K fp16 <= 128 KiB), otherwise fragments are read through L2.
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kALdsBytes = 144 * 1024;     // LDS a workgroup may take for activations + reduction (of 160 KiB)

// 4 int8 (one dword) -> 4 fp16 in two dwords, exact.
__device__ __forceinline__ void cvt4(uint32_t w, uint32_t& lo, uint32_t& hi) {
  const uint32_t b = w ^ 0x80808080u;                         // bytes now w + 128 in [1, 255]
  // v_perm_b32 byte selectors: 0..3 pick bytes of the second source, 4..7 of the first.
  uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, b, 0x07010700u);   // {0x64, b1, 0x64, b0}
  uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, b, 0x07030702u);   // {0x64, b3, 0x64, b2}
  const f16x2 bias = {(f16)1152.0f, (f16)1152.0f};
  f16x2 h0 = *reinterpret_cast<f16x2*>(&p0) - bias;
  f16x2 h1 = *reinterpret_cast<f16x2*>(&p1) - bias;
  lo = *reinterpret_cast<uint32_t*>(&h0);
  hi = *reinterpret_cast<uint32_t*>(&h1);
}

// 16 int8 -> two 8-element fp16 fragments (bytes 0..7 and 8..15).
__device__ __forceinline__ void cvt16(const u32x4& w, f16x8& f0, f16x8& f1) {
  union { uint32_t u[4]; f16x8 f; } a, b;
  cvt4(w[0], a.u[0], a.u[1]);
  cvt4(w[1], a.u[2], a.u[3]);
  cvt4(w[2], b.u[0], b.u[1]);
  cvt4(w[3], b.u[2], b.u[3]);
  f0 = a.f;
  f1 = b.f;
}

// MT: number of 16-row activation tiles handled per pass (rows m_base .. m_base + 16*MT).
template <int MT, bool A_IN_LDS>
__global__ __launch_bounds__(kThreads)
void w8a16_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                  f16* __restrict__ C, int M, int N, int K, int m_base, int n_tiles) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // [16*MT][K + 8] when A_IN_LDS: the 16-byte pad per row moves consecutive rows to consecutive bank groups
  f16* a_lds = reinterpret_cast<f16*>(smem);
  const int KP = K + 8;
  float* red = reinterpret_cast<float*>(smem + (A_IN_LDS ? (size_t)16 * MT * KP * 2 : 0));   // [kWaves][MT][256]

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r16 = lane % 16, kg = lane / 16;                               // tile row / 16-byte k group of this lane

  if constexpr (A_IN_LDS) {
    const int chunks_per_row = K / 8;
    for (int idx = threadIdx.x; idx < 16 * MT * chunks_per_row; idx += kThreads) {
      const int r = idx / chunks_per_row, c = idx % chunks_per_row;
      const int gm = m_base + r;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (gm < M) v = *reinterpret_cast<const u32x4*>(A + (int64_t)gm * K + c * 8);
      *reinterpret_cast<u32x4*>(a_lds + (int64_t)r * KP + c * 8) = v;
    }
    __syncthreads();
  }

  // K is cut into 64-wide steps (one 16-byte weight load per lane = two MFMAs). A wave takes steps in
  // adjacent pairs so that its loads cover whole 128-byte lines of each weight row: pair p = steps 2p, 2p+1,
  // wave w owns pairs w, w+8, ...
  const int steps = K / 64;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int n = tile * 16 + r16;
    const int nc = n < N ? n : N - 1;
    const int8_t* wrow = W + (int64_t)nc * K + kg * 16;
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int p0 = wave; 2 * p0 < steps; p0 += kWaves * 2) {
      u32x4 wv[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = 2 * (p0 + (u / 2) * kWaves) + (u % 2);
        wv[u] = u32x4{0u, 0u, 0u, 0u};
        if (s < steps) wv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + (int64_t)s * 64));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int s = 2 * (p0 + (u / 2) * kWaves) + (u % 2);
        if (s < steps) {
          f16x8 w0, w1;
          cvt16(wv[u], w0, w1);
          const int k = s * 64 + kg * 16;
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            f16x8 a0, a1;
            if constexpr (A_IN_LDS) {
              const f16* ap = a_lds + (int64_t)(t * 16 + r16) * KP + k;
              a0 = *reinterpret_cast<const f16x8*>(ap);
              a1 = *reinterpret_cast<const f16x8*>(ap + 8);
            } else {
              const int gm = m_base + t * 16 + r16;
              if (gm < M) {
                const f16* ap = A + (int64_t)gm * K + k;
                a0 = *reinterpret_cast<const f16x8*>(ap);
                a1 = *reinterpret_cast<const f16x8*>(ap + 8);
              } else {
                a0 = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
                a1 = a0;
              }
            }
            // D[i = channel][j = activation row]: lane holds row j = lane%16, channels 4*(lane/16) + 0..3
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, a0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, a1, acc[t], 0, 0, 0);
          }
        }
      }
    }

    // sum the K-partials of the 8 waves
#pragma unroll
    for (int t = 0; t < MT; ++t)
      *reinterpret_cast<f32x4*>(red + ((wave * MT + t) * 64 + lane) * 4) = acc[t];
    __syncthreads();
    for (int idx = threadIdx.x; idx < MT * 64; idx += kThreads) {
      const int t = idx / 64, l = idx % 64;
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum += *reinterpret_cast<const f32x4*>(red + ((w * MT + t) * 64 + l) * 4);
      const int gm = m_base + t * 16 + l % 16;
      const int gn = tile * 16 + (l / 16) * 4;
      if (gm < M) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (gn + e < N) C[(int64_t)gm * N + gn + e] = (f16)(sum[e] * (float)scales[gn + e]);
      }
    }
    __syncthreads();
  }
}

__global__ __launch_bounds__(256)
void dequant_kernel(const int8_t* __restrict__ W, const f16* __restrict__ scales, float* __restrict__ out,
                    int64_t N, int64_t K) {
  const int64_t total = N * K;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t n = i / K;
    out[i] = (float)W[i] * (float)scales[n];          // int8 -> fp32 exact, then one fp32 multiply
  }
}

template <int MT>
int launch_pass(const f16* A, const int8_t* W, const f16* s, f16* C, int M, int N, int K, int m_base, int cus,
                hipStream_t st) {
  const int n_tiles = (N + 15) / 16;
  const size_t a_bytes = (size_t)16 * MT * (K + 8) * 2;
  const size_t red_bytes = (size_t)kWaves * MT * 256 * 4;
  const bool in_lds = a_bytes + red_bytes <= (size_t)kALdsBytes;
  int grid = n_tiles < cus * 2 ? n_tiles : cus * 2;
  if (in_lds) {
    if (grid > cus) grid = cus;                       // one resident workgroup per CU (LDS bound)
    auto kern = w8a16_kernel<MT, true>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)(a_bytes + red_bytes)) != hipSuccess)
      return HEXMI_ELAUNCH;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), a_bytes + red_bytes, st, A, W, s, C, M, N, K, m_base, n_tiles);
  } else {
    hipLaunchKernelGGL((w8a16_kernel<MT, false>), dim3(grid), dim3(kThreads), red_bytes, st, A, W, s, C, M, N, K,
                       m_base, n_tiles);
  }
  return launch_status();
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" int hexmi_gemm_w8a16(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* W, const void* scales,
                                void* C, hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!A || !W || !scales || !C) return HEXMI_EINVAL;
  if (K == 0 || K % 64 != 0) return HEXMI_ENOTSUP;    // 16-byte weight loads, 64-wide K steps
  if (!aligned_to(A, 16) || !aligned_to(W, 16)) return HEXMI_EINVAL;
  if (M > 0x7fffffff || N > 0x7fffffff - 16 || K > 0x7fffffff) return HEXMI_ENOTSUP;
  int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  hipStream_t st = as_stream(stream);
  const f16* a = static_cast<const f16*>(A);
  const f16* s = static_cast<const f16*>(scales);
  f16* c = static_cast<f16*>(C);
  int rc = HEXMI_OK;
  for (int64_t m = 0; m < M && rc == HEXMI_OK; m += 64) {
    const int64_t left = M - m;
    if (left > 32) rc = launch_pass<4>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, cus, st);
    else if (left > 16) rc = launch_pass<2>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, cus, st);
    else rc = launch_pass<1>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, cus, st);
  }
  return rc;
}

extern "C" int hexmi_dequant_w8(int64_t N, int64_t K, const int8_t* W, const void* scales, float* out,
                                hexmi_stream_t stream) {
  if (N < 0 || K < 0) return HEXMI_EINVAL;
  if (N == 0 || K == 0) return HEXMI_OK;
  if (!W || !scales || !out) return HEXMI_EINVAL;
  const int64_t total = N * K;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), W,
                     static_cast<const f16*>(scales), out, N, K);
  return launch_status();
}
