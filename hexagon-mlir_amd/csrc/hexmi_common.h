// Shared device/host helpers for the hexmi kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "hexmi.h"

namespace hexmi {

constexpr int kWave = 64;  // CDNA wavefront width

typedef _Float16 f16;
typedef __bf16 bf16;

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));

// ---- scalar conversions -------------------------------------------------
template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<f16>(f16 v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<bf16>(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ f16 from_f32<f16>(float v) { return (f16)v; }   // round-to-nearest-even
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }  // round-to-nearest-even

// ---- wavefront reductions -----------------------------------------------
// Butterfly over the 64 lanes; every lane ends with the full result.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// ---- host helpers ---------------------------------------------------------
inline hipStream_t as_stream(hexmi_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? HEXMI_OK : HEXMI_ELAUNCH;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int dtype_size(int dtype) {
  switch (dtype) {
    case HEXMI_F32: return 4;
    case HEXMI_F16: case HEXMI_BF16: return 2;
    case HEXMI_I8: return 1;
    default: return 0;
  }
}

}  // namespace hexmi
