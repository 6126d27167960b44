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

// four consecutive elements, rounded once to the output type, in one store (p aligned to 4 elements)
template <typename OutT>
__device__ __forceinline__ void store4(OutT* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
  f32x4 v = {a, b, c, d};
  *reinterpret_cast<f32x4*>(p) = v;
}
template <> __device__ __forceinline__ void store4<f16>(f16* p, float a, float b, float c, float d) {
  f16x4 v = {(f16)a, (f16)b, (f16)c, (f16)d};
  *reinterpret_cast<f16x4*>(p) = v;
}
template <> __device__ __forceinline__ void store4<bf16>(bf16* p, float a, float b, float c, float d) {
  bf16x4 v = {(bf16)a, (bf16)b, (bf16)c, (bf16)d};
  *reinterpret_cast<bf16x4*>(p) = v;
}

// ---- wavefront reductions -----------------------------------------------
// Butterfly over the 64 lanes on the vector ALU (no LDS round trips): DPP exchanges inside a row of 16 lanes
// (quad permutes for lane^1 and lane^2; the half-row and row mirrors stand in for lane^4 and lane^8 because the
// partial results are already uniform inside groups of 4 and 8), then v_permlane16_swap / v_permlane32_swap
// for the exchanges between rows. Every lane ends with the full result.
// (Every lane has a valid source under these permutations, so the value for lanes without one is never used; it is
// given as 0 with the bound-control bit set, the form the compiler folds into the add or max that consumes the
// exchange - v_add_f32_dpp, one instruction per step - where "keep the own value" leaves a copy, the exchange and
// the add: three.)
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  const int i = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, CTRL, 0xF, 0xF, true));
}
// {a, b} with a = value of the partner row (16 lanes) / half (32 lanes) and b = own, in some order that is the
// same for both partners up to exchange: callers combine them with a commutative operation.
__device__ __forceinline__ void swap16(float v, float& a, float& b) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  a = __builtin_bit_cast(float, (unsigned)r[0]);
  b = __builtin_bit_cast(float, (unsigned)r[1]);
}
__device__ __forceinline__ void swap32(float v, float& a, float& b) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  a = __builtin_bit_cast(float, (unsigned)r[0]);
  b = __builtin_bit_cast(float, (unsigned)r[1]);
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1>(v);      // quad_perm [1,0,3,2]
  v += dpp_move<0x4E>(v);      // quad_perm [2,3,0,1]
  v += dpp_move<0x141>(v);     // row_half_mirror
  v += dpp_move<0x140>(v);     // row_mirror
  float a, b;
  swap16(v, a, b);
  v = a + b;
  swap32(v, a, b);
  return a + b;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1>(v));
  v = fmaxf(v, dpp_move<0x4E>(v));
  v = fmaxf(v, dpp_move<0x141>(v));
  v = fmaxf(v, dpp_move<0x140>(v));
  float a, b;
  swap16(v, a, b);
  v = fmaxf(a, b);
  swap32(v, a, b);
  return fmaxf(a, b);
}

// ---- int8 -> fp16 (weight-only quantisation) --------------------------------
// 4 int8 (one dword) -> 4 fp16 in two dwords, exact (|w| <= 128 has at most eight significant bits): one
// v_cvt_f16_i16 per weight, its source the sign-extended byte picked by the instruction's operand selector and its
// destination one half of the result register. (One instruction fewer per dword than building 1024 + (w ^ 0x80) with
// byte permutes and subtracting 1152 in packed fp16: 0.157 -> 0.164 of the HBM figure at M = 256, +1 % at M = 1.)
__device__ __forceinline__ void cvt4(uint32_t w, uint32_t& lo, uint32_t& hi) {
  asm("v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t"
      "v_cvt_f16_i16_sdwa %0, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1\n\t"
      "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t"
      "v_cvt_f16_i16_sdwa %1, sext(%2) dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3"
      : "=&v"(lo), "=&v"(hi)
      : "v"(w));
}

// 16 int8 -> two 8-element fp16 fragments (bytes 0..7 and 8..15), as ONE statement that ends in two idle issue
// slots. A matrix instruction must not read a register in the two slots after a vector instruction wrote it, and
// the compiler, which keeps that distance for its own instructions, cannot see the writes inside an asm statement:
// with a conversion one slot ahead of its MFMA, and the matrix pipe still busy with the MFMA before, the MFMA read
// the register without the last converted byte (k = 11 mod 16 lost in every product; one slot was enough wherever
// the pipe was idle). Callers of cvt4 keep the distance themselves.
__device__ __forceinline__ void cvt16(const u32x4& w, f16x8& f0, f16x8& f1) {
  union { uint32_t u[4]; f16x8 f; } a, b;
#define HEXMI_CVT4(LO, HI, SRC) \
      "v_cvt_f16_i16_sdwa " LO ", sext(" SRC ") dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_0\n\t" \
      "v_cvt_f16_i16_sdwa " LO ", sext(" SRC ") dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_1\n\t" \
      "v_cvt_f16_i16_sdwa " HI ", sext(" SRC ") dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:BYTE_2\n\t" \
      "v_cvt_f16_i16_sdwa " HI ", sext(" SRC ") dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:BYTE_3\n\t"
  asm(HEXMI_CVT4("%0", "%1", "%8") HEXMI_CVT4("%2", "%3", "%9") HEXMI_CVT4("%4", "%5", "%10")
      HEXMI_CVT4("%6", "%7", "%11") "s_nop 1"
      : "=&v"(a.u[0]), "=&v"(a.u[1]), "=&v"(a.u[2]), "=&v"(a.u[3]), "=&v"(b.u[0]), "=&v"(b.u[1]), "=&v"(b.u[2]),
        "=&v"(b.u[3])
      : "v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]));
#undef HEXMI_CVT4
  f0 = a.f;
  f1 = b.f;
}

// ---- host helpers ---------------------------------------------------------
inline hipStream_t as_stream(hexmi_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Every entry point calls begin_call() once its arguments are accepted and before its first launch: HIP keeps one
// pending error per host thread, and one left there by unrelated code would otherwise be reported (and cleared) by
// the launch_status() of the next launch here.
inline void begin_call() { (void)hipGetLastError(); }

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? HEXMI_OK : HEXMI_ELAUNCH;
}

// C[rows, cols] = 0 with leading dimension ld (elements of elem_size bytes): what a product over an empty inner
// dimension is (gemm.hip).
int fill_zero_2d(void* C, int64_t rows, int64_t cols, int64_t ld, int elem_size, hipStream_t stream);

// 16 bytes per lane, global -> LDS, as a buffer load: the address is a uniform base (a buffer descriptor in scalar
// registers, built by scalar arithmetic) plus a per-lane 32-bit byte offset, and the LDS destination (lds + lane*16
// bytes) is a scalar, so a copy costs no vector arithmetic. voff must stay below 2^31; the descriptor's own range
// check is left wide open, callers clamp what must not be read.
// POLICY: the cache-policy bits of the load (0 = default, 2 = non-temporal: data that is read once).
template <typename T, int POLICY = 0>
__device__ __forceinline__ void copy_to_lds(const char* base, int voff, T* lds) {
#if defined(__HIP_DEVICE_COMPILE__)        // the descriptor type exists in the device pass only
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, 0x7fffffff, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(lds), 16, voff, 0, 0, POLICY);
#endif
}

// copy_to_lds written as asm, for kernels whose LDS destination the compiler cannot name (a stage picked at run
// time, a wave-private region at a run-time base): a copy into LDS with an unknown target makes the compiler wait
// for ALL copies in flight (vmcnt(0)) before every later LDS read that might alias it. A kernel that uses this for
// its copies does its own waiting (s_waitcnt vmcnt) before reading what they fill: the compiler does not know the
// copies exist. Its own vmcnt waits for other loads only get stronger (the counter counts these copies too, and
// loads complete in issue order). M0 (the LDS destination of such a copy) is saved and restored because the
// compiler tracks its own uses of it. lds must be wave-uniform.
template <typename T>
__device__ __forceinline__ void copy_to_lds_asm(const char* base, int voff, T* lds) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef int i32x4_rsrc __attribute__((ext_vector_type(4)));
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  i32x4_rsrc rsrc;
  rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
  rsrc[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(b >> 32) & 0xffffu));
  rsrc[2] = 0x7fffffff;
  rsrc[3] = 0x00020000;
  const uint32_t dst = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)(lds)));
  uint32_t saved;
  asm volatile(
      "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
      "buffer_load_dwordx4 %2, %3, 0 offen lds\n\ts_mov_b32 m0, %0"
      : "=&s"(saved)
      : "s"(dst), "v"(voff), "s"(rsrc)
      : "memory");
#endif
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

// Block sums (elementwise.hip). A program of kTwoPassMinBlock elements and more is summed in two passes when a
// scratch buffer for fp32 partial sums of runs of kSumRun elements is at hand (ceil(n / kSumRun) floats): the runs of
// a program must be whole, which they are when block % kSumRun == 0 or there is a single program.
constexpr int64_t kSumRun = 4096;
constexpr int64_t kTwoPassMinBlock = 1 << 16;
inline bool two_pass_sum(int64_t n, int64_t block) {
  const int64_t programs = (n + block - 1) / block;
  return block >= kTwoPassMinBlock && (programs == 1 || block % kSumRun == 0);
}
// partials == nullptr: one pass; otherwise two_pass_sum(n, block) holds and partials has room for every run.
int block_sum_any(const void* x, void* out, int64_t n, int64_t block, int dtype, float* partials, hipStream_t s);

// Tiled W8A16 GEMM for many activation rows (gemm.hip): C[M,N] = (A[M,K] * W[N,K]^T) * scales[N].
int gemm_w8a16_tiled(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales, f16* C,
                     hipStream_t stream);
int gemm_w8a16_any_shape(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales,
                         const int8_t* zero_points, int per_tensor, f16* C, hipStream_t stream);

// W8A16 on a (channel range x K part) decomposition with the K parts summed through a caller workspace
// (w8a16_split.hip). w8a16_split_workspace: bytes the shape needs (0: one K part, or a shape the kernel does not
// take). w8a16_split returns false when it does not take the call (shape, alignment, workspace too small).
int64_t w8a16_split_workspace(int64_t M, int64_t N, int64_t K, int cus);
int64_t w8a16_split_header(int64_t M, int64_t N, int64_t K, int cus);   // leading bytes that must be zero at launch
bool w8a16_split(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales, f16* C,
                 void* workspace, int64_t workspace_bytes, int cus, hipStream_t stream, int* status);
// zeroes the first `bytes` of a workspace (a kernel, not a memset: callers may be under graph capture)
int w8a16_split_clear(void* workspace, int64_t bytes, hipStream_t stream);

// fp32 GEMM on the matrix cores (gemm_f32.hip): launches and returns true when the shapes fit (K % 32 == 0, aligned
// operands), with the launch status in *status; false leaves the product to the vector-ALU kernel.
bool gemm_f32_mfma(bool trans_b, const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, hipStream_t stream, int* status);

// fp32 flash attention on the fp32 matrix cores (flash_attn_f32.hip): launches and returns true when the shapes fit
// (head size 64 or 128, aligned operands), with the launch status in *status.
bool flash_attn_f32_mfma(const float* Q, const float* K, const float* V, const float* mask, float* O, int64_t ZH,
                         int64_t S, int64_t Skv, int64_t D, float scale_log2e, bool causal, hipStream_t stream,
                         int* status);

}  // namespace hexmi
