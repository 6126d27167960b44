// Measurement aid: what the matrix cores of this GPU sustain on a stream of nothing but MFMAs (operands and
// accumulators in registers, no memory traffic), for the two instruction shapes the kernels here use and for
// operands of the caller's choice. The rate depends on the data: the chip is power-limited, all-zero operands
// toggle nothing and hold the top clock, random operands do not. Roofline fractions of the MFMA-bound kernels are
// priced against the published peak; this figure says how much of that peak any kernel could reach on such data.
#include "hexmi_common.h"

namespace hexmi {
namespace {

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <typename T> struct Peak;
template <> struct Peak<f16> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x16 big(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ f32x4v small(Frag a, Frag b, f32x4v c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct Peak<bf16> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x16 big(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ f32x4v small(Frag a, Frag b, f32x4v c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

constexpr int kBigChains = 4;      // independent accumulators: 32x32x16, 64 registers
constexpr int kSmallChains = 8;    // 16x16x32, 32 registers
constexpr int kUnroll = 4;         // rounds over all chains per loop iteration

// operands: 2 KiB, lane l reads its A fragment at byte 16*l and its B fragment at byte 1024 + 16*l.
template <typename T, bool BIG>
__global__ __launch_bounds__(512)
void mfma_peak_kernel(const T* __restrict__ operands, int iters, float* __restrict__ sink) {
  typedef typename Peak<T>::Frag Frag;
  const int lane = threadIdx.x % kWave;
  const Frag a = *reinterpret_cast<const Frag*>(operands + lane * 8);
  const Frag b = *reinterpret_cast<const Frag*>(operands + 512 + lane * 8);
  float total = 0.0f;
  if constexpr (BIG) {
    f32x16 acc[kBigChains];
#pragma unroll
    for (int c = 0; c < kBigChains; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int c = 0; c < kBigChains; ++c) acc[c] = Peak<T>::big(a, b, acc[c]);
    }
#pragma unroll
    for (int c = 0; c < kBigChains; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) total += acc[c][r];
  } else {
    f32x4v acc[kSmallChains];
#pragma unroll
    for (int c = 0; c < kSmallChains; ++c) acc[c] = f32x4v{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
#pragma unroll
        for (int c = 0; c < kSmallChains; ++c) acc[c] = Peak<T>::small(a, b, acc[c]);
    }
#pragma unroll
    for (int c = 0; c < kSmallChains; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) total += acc[c][r];
  }
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = total;
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" double hexmi_mfma_peak_flops(int shape, int waves_per_simd, int64_t iters) {
  const int cus = hexmi_num_cus();
  if (cus <= 0 || (shape != 0 && shape != 1) || waves_per_simd < 1 || waves_per_simd > 2 || iters < 0) return 0.0;
  const double per_wave_iter = shape == 0 ? (double)kUnroll * kBigChains * (2.0 * 32 * 32 * 16)
                                          : (double)kUnroll * kSmallChains * (2.0 * 16 * 16 * 32);
  return per_wave_iter * (double)iters * 4.0 * waves_per_simd * cus;
}

extern "C" int hexmi_mfma_peak(int shape, int dtype, const void* operands, int64_t iters, int waves_per_simd,
                               float* sink, hexmi_stream_t stream) {
  if ((shape != 0 && shape != 1) || waves_per_simd < 1 || waves_per_simd > 2 || iters < 0 || iters > 0x7fffffff)
    return HEXMI_EINVAL;
  if (!operands || !sink || !aligned_to(operands, 16)) return HEXMI_EINVAL;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  hipStream_t st = as_stream(stream);
  const dim3 grid((unsigned)cus), block(256u * waves_per_simd);
  begin_call();
#define HEXMI_PEAK(T, BIG) \
  hipLaunchKernelGGL((mfma_peak_kernel<T, BIG>), grid, block, 0, st, static_cast<const T*>(operands), (int)iters, sink)
  if (dtype == HEXMI_F16) { if (shape == 0) HEXMI_PEAK(f16, true); else HEXMI_PEAK(f16, false); }
  else if (dtype == HEXMI_BF16) { if (shape == 0) HEXMI_PEAK(bf16, true); else HEXMI_PEAK(bf16, false); }
  else return HEXMI_ENOTSUP;
#undef HEXMI_PEAK
  return launch_status();
}
