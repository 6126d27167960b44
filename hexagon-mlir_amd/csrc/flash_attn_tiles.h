// Pieces of the 16-bit flash-attention kernels (flash_attn.hip): MFMA wrappers, the
// swizzled [64 keys][D] LDS tile and its global -> LDS loader, half-wave exchange, 4-element stores.
#pragma once
#include "hexmi_common.h"

namespace hexmi {
namespace {

#define HEXMI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define HEXMI_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int kWideMinS = 2048;  // sequences at least this long may use 8-wave (256-row) workgroups
constexpr int kBlockN = 64;    // keys per step
constexpr float kRescaleLag = 8.0f;   // how far (log2) the softmax reference maximum may trail the true one

template <typename T> struct MfmaT;
template <> struct MfmaT<f16> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ Frag pack(const float* p) {
    return Frag{(f16)p[0], (f16)p[1], (f16)p[2], (f16)p[3], (f16)p[4], (f16)p[5], (f16)p[6], (f16)p[7]};
  }
  // acc + the eight packed values, two per instruction
  static __device__ __forceinline__ float sum8(Frag f, float acc) {
    const f16x2 one = {(f16)1.0f, (f16)1.0f};
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_fdot2(f16x2{f[2 * e], f[2 * e + 1]}, one, acc, false);
    return acc;
  }
};
template <> struct MfmaT<bf16> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ Frag pack(const float* p) {
    return Frag{(bf16)p[0], (bf16)p[1], (bf16)p[2], (bf16)p[3], (bf16)p[4], (bf16)p[5], (bf16)p[6], (bf16)p[7]};
  }
  static __device__ __forceinline__ float sum8(Frag f, float acc) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const bf16x2_t one = {(bf16)1.0f, (bf16)1.0f};
#pragma unroll
    for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2_t{f[2 * e], f[2 * e + 1]}, one, acc, false);
    return acc;
  }
};

// LDS tile [64 keys][D], 16-byte chunks, XOR swizzled per row. K is read with ds_read_b128 by 32 rows at one
// chunk position; V with transposing 8-byte reads that touch 8 rows x 64 bytes.
template <int D> __device__ __forceinline__ int swz_ktile(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
template <int D> __device__ __forceinline__ int swz_vtile(int row) {
  return D == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

// global -> LDS copy of one [64 keys][D] tile: 64*D/8/64/4 wave-wide instructions per wave. The per-lane element
// offsets inside a tile do not change from tile to tile, so they are computed once; only a ragged last tile
// (keys past the end of the sequence) needs its rows clamped.
// PADDED: the head is narrower than the tile (d % 8 == 0, d < D): rows are d elements apart in memory, and a lane
// whose chunk lies past column d copies nothing -- its LDS positions, which no other lane ever writes, are zeroed
// once by the kernel (zero_padding), so the tile reads as the head padded with zero columns.
template <typename T, int D, bool IS_V, int NW = 4, bool PADDED = false>
struct KvTileLoader {
  static constexpr int CPR = D / 8;                       // chunks per row
  static constexpr int NI = kBlockN * CPR / 64 / NW;      // instructions per wave
  static constexpr int kRowsPerInst = 64 / CPR;           // rows one wave-wide instruction covers
  static constexpr int kRowStep = NW * kRowsPerInst;      // rows between this wave's instructions j and j+1
  // The swizzles repeat every 16 rows (32 for D = 64) and kRowStep is a multiple of that, so instruction j reads
  // the lane's chunk of instruction 0 moved down by j*kRowStep rows: one offset, one row and one column per lane.
  static_assert(kRowStep % (D == 128 ? 16 : 32) == 0, "swizzle period");
  int off0;                                               // element offset of this lane's chunk inside a tile, j = 0
  int row0, col0;
  int lds_off0;
  int d;                                                  // elements between rows in memory (D unless PADDED)
  bool live;                                              // this lane's chunk is inside the head
  // live_cols: columns of the tile that exist in memory (the head itself, or what is left of it for a tile that
  // starts at a column offset: the caller then passes the offset pointer)
  __device__ __forceinline__ void init(int wave, int lane, int head_dim = D, int live_cols = D) {
    const int lin = wave * 64 + lane;
    row0 = lin / CPR;
    col0 = ((lin % CPR) ^ (IS_V ? swz_vtile<D>(row0) : swz_ktile<D>(row0))) * 8;
    d = PADDED ? head_dim : D;
    live = !PADDED || col0 < live_cols;
    off0 = row0 * d + col0;
    lds_off0 = wave * 64 * 8;
  }
  // PADDED: zeros where this lane would have copied, in one stage
  __device__ __forceinline__ void zero_padding(T* lds, int lane) const {
    if (!live) {
#pragma unroll
      for (int j = 0; j < NI; ++j)
        *reinterpret_cast<u32x4*>(lds + lds_off0 + j * (NW * 64 * 8) + lane * 8) = u32x4{0u, 0u, 0u, 0u};
    }
  }
  // instruction j of this wave's share of a tile that lies wholly inside the sequence
  __device__ __forceinline__ void issue_one_whole(int j, const T* __restrict__ g, int key0, T* lds) const {
    const char* base = reinterpret_cast<const char*>(g + ((int64_t)key0 + j * kRowStep) * d);
    if (live) copy_to_lds(base, off0 * (int)sizeof(T), lds + lds_off0 + j * (NW * 64 * 8));
  }
  // instruction j of this wave's share of the tile
  __device__ __forceinline__ void issue_one(int j, const T* __restrict__ g, int key0, int S, T* lds) const {
    T* dst = lds + lds_off0 + j * (NW * 64 * 8);
    if (key0 + kBlockN <= S) {
      issue_one_whole(j, g, key0, lds);
    } else {
      // ragged last tile: rows clamped to the last key, offsets from the head's first key (S*D*sizeof(T) < 2^31)
      const char* base = reinterpret_cast<const char*>(g);
      int key = key0 + row0 + j * kRowStep;
      key = key < S ? key : S - 1;
      if (live) copy_to_lds(base, (key * d + col0) * (int)sizeof(T), dst);
    }
  }
  __device__ __forceinline__ void issue(const T* __restrict__ g, int key0, int S, T* lds) const {
#pragma unroll
    for (int j = 0; j < NI; ++j) issue_one(j, g, key0, S, lds);
  }
};

// Value held by lane ^ 32 (v_permlane32_swap exchanges the upper half of one register with the lower half of
// another; no LDS round trip).
__device__ __forceinline__ float other_half(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned lo = r[0], hi = r[1];              // lo: lanes hold v[lane%32], hi: lanes hold v[lane%32 + 32]
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? lo : hi);
}

template <typename OutT>
__device__ __forceinline__ void store4o(OutT* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4o<float>(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<f32x4*>(p) = f32x4{a, b, c, d};
}
template <> __device__ __forceinline__ void store4o<f16>(f16* p, float a, float b, float c, float d) {
  *reinterpret_cast<f16x4*>(p) = f16x4{(f16)a, (f16)b, (f16)c, (f16)d};
}
template <> __device__ __forceinline__ void store4o<bf16>(bf16* p, float a, float b, float c, float d) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)a, (bf16)b, (bf16)c, (bf16)d};
}

}  // namespace
}  // namespace hexmi
