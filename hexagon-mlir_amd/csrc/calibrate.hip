// Measurement aid: what the matrix cores of this GPU sustain on a stream of nothing but MFMAs (operands and
// accumulators in registers, no memory traffic), for the two instruction shapes the kernels here use and for
// operands of the caller's choice. The rate depends on the data: the chip is power-limited, all-zero operands
// toggle nothing and hold the top clock, random operands do not. Roofline fractions of the MFMA-bound kernels are
// priced against the published peak; this figure says how much of that peak any kernel could reach on such data.
#include <type_traits>

#include "hexmi_common.h"
#include "hexmi_calibrate.h"

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


// The same stream with the operands of a GEMM tile: 8 x 8 accumulator tiles of 16x16x32 per wave (one wave per SIMD,
// 256 accumulator registers), accumulator (i, j) fed by A fragment i and B fragment j, walked row by row, so one
// operand changes with every instruction and the other with every eighth, as in gemm.hip. operands: 16 KiB, A
// fragment i of lane l at byte 1024*i + 16*l, B fragment j at byte 8192 + 1024*j + 16*l.
template <typename T>
__global__ __launch_bounds__(256)
void mfma_tile_kernel(const T* __restrict__ operands, int iters, float* __restrict__ sink) {
  typedef typename Peak<T>::Frag Frag;
  const int lane = threadIdx.x % kWave;
  Frag a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = *reinterpret_cast<const Frag*>(operands + (i * 64 + lane) * 8);
    b[i] = *reinterpret_cast<const Frag*>(operands + 4096 + (i * 64 + lane) * 8);
  }
  f32x4v acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = f32x4v{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = Peak<T>::small(b[j], a[i], acc[i][j]);
  }
  float total = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) total += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = total;
}

// ---- issue slots --------------------------------------------------------------------------------------------
// How much vector work fits under a wave's own MFMAs: per MFMA (independent accumulators, zero operands, so the chip
// holds its top clock) VPM vector instructions of one kind follow in the same instruction stream. A SIMD issues one
// instruction at a time, so the time per MFMA is the larger of the matrix pipe's (16 or 32 cycles) and the issue time
// of everything in between.
template <bool BIG, int KIND, int VPM>
__global__ __launch_bounds__(512)
void issue_slots_kernel(int iters, float* __restrict__ sink) {
  const f16x8 a = {0, 0, 0, 0, 0, 0, 0, 0}, b = a;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = 0.001f * (float)(threadIdx.x + i);
  constexpr int NM = BIG ? 4 : 16;                 // 64 accumulator registers either way
  typedef typename std::conditional<BIG, f32x16, f32x4v>::type Acc;
  Acc acc[NM];
#pragma unroll
  for (int m = 0; m < NM; ++m)
#pragma unroll
    for (int r = 0; r < (BIG ? 16 : 4); ++r) acc[m][r] = 0.0f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      if constexpr (BIG) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[m]) : "v"(a), "v"(b));
      else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[m]) : "v"(a), "v"(b));
#pragma unroll
      for (int n = 0; n < VPM; ++n) {
        const int idx = (m * VPM + n) % 8;         // eight independent chains
        if constexpr (KIND == 0) asm volatile("v_pk_add_f16 %0, %0, %0" : "+v"(v[idx]));
        else if constexpr (KIND == 1) asm volatile("v_fma_f32 %0, %0, %0, %0" : "+v"(v[idx]));
        else if constexpr (KIND == 2) asm volatile("v_exp_f32 %0, %0" : "+v"(v[idx]));
        else if constexpr (KIND == 3) asm volatile("v_fma_mix_f32 %0, %0, %0, %0 op_sel_hi:[1,0,0]" : "+v"(v[idx]));
        else asm volatile("v_cvt_f32_f16 %0, %0" : "+v"(v[idx]));
      }
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the MFMAs are assembly: wait states before reading acc
  float total = 0.0f;
#pragma unroll
  for (int m = 0; m < NM; ++m) total += acc[m][0];
#pragma unroll
  for (int i = 0; i < 8; ++i) total += v[i];
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = total;
}

template <bool BIG, int KIND>
int launch_issue_slots(int per_mfma, dim3 grid, dim3 block, hipStream_t st, int iters, float* sink) {
#define HEXMI_SLOTS(V) case V: hipLaunchKernelGGL((issue_slots_kernel<BIG, KIND, V>), grid, block, 0, st, iters, sink); break;
  switch (per_mfma) {
    HEXMI_SLOTS(0) HEXMI_SLOTS(1) HEXMI_SLOTS(2) HEXMI_SLOTS(3) HEXMI_SLOTS(4) HEXMI_SLOTS(5) HEXMI_SLOTS(6) HEXMI_SLOTS(8)
    default: return HEXMI_EINVAL;
  }
#undef HEXMI_SLOTS
  return launch_status();
}

// ---- LDS read patterns --------------------------------------------------------------------------------------
// Cycles per wave-wide ds_read_b128 for the fragment-read address patterns of the tiled GEMM, with 16 waves per
// compute unit issuing nothing else (the LDS saturated). Eight reads (four 16-row tiles x two K steps) per round.
// 0 lane*16 (linear)                    3 the same read with swizzle ((r>>1)&1) | ((r&1)<<1) | (r&4)
// 1 fp16 rows of 128 bytes, lane group g reads chunk 4*step + g, chunks XOR-swizzled by (row >> 1) & 7
// 2 the same rows read as chunk 2*g + step (what int8 B imposes on A), same swizzle
// 4 int8 rows of 64 bytes, lane group g reads chunk g, swizzle (row >> 2) & 3      5 the same, swizzle (row >> 1) & 3
// 6 pattern 1 without a swizzle
__device__ __forceinline__ int lds_pattern_addr(int pattern, int lane, int t) {
  const int r16 = lane % 16, g = lane / 16, step = t / 4;
  const int row = (t % 4) * 16 + r16;
  switch (pattern) {
    case 0: return t * 1024 + lane * 16;
    case 1: return row * 128 + (((4 * step + g) ^ ((row >> 1) & 7)) * 16);
    case 2: return row * 128 + (((2 * g + step) ^ ((row >> 1) & 7)) * 16);
    case 3: return row * 128 + (((2 * g + step) ^ (((row >> 1) & 1) | ((row & 1) << 1) | (row & 4))) * 16);
    case 4: return (t * 16 + r16) * 64 + ((g ^ (((t * 16 + r16) >> 2) & 3)) * 16);
    case 5: return (t * 16 + r16) * 64 + ((g ^ (((t * 16 + r16) >> 1) & 3)) * 16);
    default: return row * 128 + (4 * step + g) * 16;
  }
}

constexpr int kLdsPatternBytes = 32768;             // four waves' worth of 8 KiB tiles

__global__ __launch_bounds__(1024)
void lds_pattern_kernel(int pattern, int iters, float* __restrict__ sink) {
  __shared__ __attribute__((aligned(16))) uint32_t tile[kLdsPatternBytes / 4];
  for (int i = threadIdx.x; i < kLdsPatternBytes / 4; i += blockDim.x) reinterpret_cast<volatile uint32_t*>(tile)[i] = i;
  __syncthreads();
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int base = (int)(uintptr_t)((__attribute__((address_space(3))) void*)tile) + (wave % 4) * 8192;
  int addr[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) addr[t] = base + lds_pattern_addr(pattern, lane, t);
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      u32x4 v;
      asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(4)" : "=v"(v) : "v"(addr[t]) : "memory");
      acc ^= v;                                   // may see the register before the read lands: only the time matters
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = (float)(acc[0] ^ acc[1] ^ acc[2] ^ acc[3]);
}


// What a compute unit can take in from L2: 16 waves per workgroup, one workgroup per CU, every wave streaming
// 1 KiB pieces of a region that stays in L2, either straight into LDS (global_load_lds, the path of the W8A16
// kernels' activation and weight copies) or into registers. `shared`: every workgroup reads the same region at
// the same time (activations: one matrix, every CU) or a region of its own. No waits inside the loop: the
// hardware's queues set the pace.
template <bool TO_LDS>
__global__ __launch_bounds__(1024)
void l2_stream_kernel(const char* __restrict__ src, int64_t region_bytes, int shared, int passes, float* __restrict__ sink) {
  __shared__ __attribute__((aligned(16))) char stage[64 << 10];
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const char* base = src + (shared ? 0 : (int64_t)blockIdx.x * region_bytes);
  const int64_t pieces = region_bytes / (16 << 10);          // 16 KiB per workgroup and step
  u32x4 keep = {0u, 0u, 0u, 0u};
  for (int p = 0; p < passes; ++p) {
    for (int64_t i = 0; i < pieces; i += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const char* at = base + ((i + u) % pieces) * (16 << 10) + wave * 1024 + lane * 16;
        if constexpr (TO_LDS) {
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)at,
                                           (__attribute__((address_space(3))) void*)(stage + u * (16 << 10) + wave * 1024), 16, 0, 0);
        } else {
          const u32x4 v = *reinterpret_cast<const u32x4*>(at);
          keep[0] ^= v[0]; keep[1] ^= v[1]; keep[2] ^= v[2]; keep[3] ^= v[3];
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  float out = (float)(keep[0] ^ keep[1] ^ keep[2] ^ keep[3]);
  if constexpr (TO_LDS) out += (float)stage[threadIdx.x * 16];
  sink[blockIdx.x * 1024 + threadIdx.x] = out;
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" double hexmi_mfma_peak_flops(int shape, int waves_per_simd, int64_t iters) {
  const int cus = hexmi_num_cus();
  if (cus <= 0 || shape < 0 || shape > 2 || waves_per_simd < 1 || waves_per_simd > (shape == 2 ? 1 : 2) || iters < 0)
    return 0.0;
  const double per_wave_iter = shape == 0 ? (double)kUnroll * kBigChains * (2.0 * 32 * 32 * 16)
                               : shape == 1 ? (double)kUnroll * kSmallChains * (2.0 * 16 * 16 * 32)
                                            : 64.0 * (2.0 * 16 * 16 * 32);
  return per_wave_iter * (double)iters * 4.0 * waves_per_simd * cus;
}

extern "C" int hexmi_mfma_peak(int shape, int dtype, const void* operands, int64_t iters, int waves_per_simd,
                               float* sink, hexmi_stream_t stream) {
  if (shape < 0 || shape > 2 || waves_per_simd < 1 || waves_per_simd > (shape == 2 ? 1 : 2) || iters < 0)
    return HEXMI_EINVAL;
  if (!operands || !sink || !aligned_to(operands, 16)) return HEXMI_EINVAL;
  if (iters > HEXMI_CALIBRATE_MAX_ITERS) return HEXMI_ETOOBIG;   // one launch holds every CU: keep it to about a minute
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  hipStream_t st = as_stream(stream);
  const dim3 grid((unsigned)cus), block(256u * waves_per_simd);
  begin_call();
  if (shape == 2) {
    if (dtype == HEXMI_F16)
      hipLaunchKernelGGL(mfma_tile_kernel<f16>, grid, block, 0, st, static_cast<const f16*>(operands), (int)iters, sink);
    else if (dtype == HEXMI_BF16)
      hipLaunchKernelGGL(mfma_tile_kernel<bf16>, grid, block, 0, st, static_cast<const bf16*>(operands), (int)iters, sink);
    else
      return HEXMI_ENOTSUP;
    return launch_status();
  }
#define HEXMI_PEAK(T, BIG) \
  hipLaunchKernelGGL((mfma_peak_kernel<T, BIG>), grid, block, 0, st, static_cast<const T*>(operands), (int)iters, sink)
  if (dtype == HEXMI_F16) { if (shape == 0) HEXMI_PEAK(f16, true); else HEXMI_PEAK(f16, false); }
  else if (dtype == HEXMI_BF16) { if (shape == 0) HEXMI_PEAK(bf16, true); else HEXMI_PEAK(bf16, false); }
  else return HEXMI_ENOTSUP;
#undef HEXMI_PEAK
  return launch_status();
}

extern "C" int hexmi_issue_slots(int shape, int kind, int per_mfma, int64_t iters, int waves_per_simd, float* sink,
                                 hexmi_stream_t stream) {
  if ((shape != 0 && shape != 1) || kind < 0 || kind > 4 || waves_per_simd < 1 || waves_per_simd > 2 || iters < 0 ||
      !sink)
    return HEXMI_EINVAL;
  if (iters > HEXMI_CALIBRATE_MAX_ITERS) return HEXMI_ETOOBIG;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  hipStream_t st = as_stream(stream);
  const dim3 grid((unsigned)cus), block(256u * waves_per_simd);
  begin_call();
  if (shape == 0) {
    if (kind == 0) return launch_issue_slots<true, 0>(per_mfma, grid, block, st, (int)iters, sink);
    if (kind == 1) return launch_issue_slots<true, 1>(per_mfma, grid, block, st, (int)iters, sink);
    if (kind == 2) return launch_issue_slots<true, 2>(per_mfma, grid, block, st, (int)iters, sink);
    if (kind == 3) return launch_issue_slots<true, 3>(per_mfma, grid, block, st, (int)iters, sink);
    return launch_issue_slots<true, 4>(per_mfma, grid, block, st, (int)iters, sink);
  }
  if (kind == 0) return launch_issue_slots<false, 0>(per_mfma, grid, block, st, (int)iters, sink);
  if (kind == 1) return launch_issue_slots<false, 1>(per_mfma, grid, block, st, (int)iters, sink);
  if (kind == 2) return launch_issue_slots<false, 2>(per_mfma, grid, block, st, (int)iters, sink);
  if (kind == 3) return launch_issue_slots<false, 3>(per_mfma, grid, block, st, (int)iters, sink);
  return launch_issue_slots<false, 4>(per_mfma, grid, block, st, (int)iters, sink);
}

extern "C" int hexmi_lds_read_pattern(int pattern, int64_t iters, float* sink, hexmi_stream_t stream) {
  if (pattern < 0 || pattern > 6 || iters < 0 || !sink) return HEXMI_EINVAL;
  if (iters > HEXMI_CALIBRATE_MAX_ITERS) return HEXMI_ETOOBIG;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  begin_call();
  hipLaunchKernelGGL(lds_pattern_kernel, dim3((unsigned)cus), dim3(1024), 0, as_stream(stream), pattern, (int)iters, sink);
  return launch_status();
}

extern "C" int hexmi_l2_stream(int to_lds, int shared, int64_t region_bytes, int64_t passes, const void* src, float* sink,
                               hexmi_stream_t stream) {
  if (region_bytes < (64 << 10) || region_bytes % (64 << 10) != 0 || passes < 0 || !src || !sink || !aligned_to(src, 16))
    return HEXMI_EINVAL;
  // at most 64 GiB through a compute unit: a few seconds at any rate worth measuring
  if (passes > HEXMI_CALIBRATE_MAX_ITERS || (double)passes * (double)region_bytes > 64.0 * (1 << 30)) return HEXMI_ETOOBIG;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  begin_call();
  if (to_lds)
    hipLaunchKernelGGL(l2_stream_kernel<true>, dim3((unsigned)cus), dim3(1024), 0, as_stream(stream),
                       static_cast<const char*>(src), region_bytes, shared, (int)passes, sink);
  else
    hipLaunchKernelGGL(l2_stream_kernel<false>, dim3((unsigned)cus), dim3(1024), 0, as_stream(stream),
                       static_cast<const char*>(src), region_bytes, shared, (int)passes, sink);
  return launch_status();
}
