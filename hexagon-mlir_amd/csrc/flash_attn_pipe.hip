// Flash-attention forward, software-pipelined inside one wave: fp16 / bf16, D = 128, S a multiple of 64, no mask.
//
// A workgroup is four waves, one per SIMD, and owns 256 query rows; a wave owns 64 of them as two 32-row tiles A
// and B that take turns on the matrix cores. Iteration i of the key loop works on V(i) and K(i+1) in two slots of one
// straight-line instruction stream:
//   slot A: matrix cores: O_A += V(i)^T P_A(i)^T, then S_A(i+1)^T = K(i+1) Q_A^T     vector ALUs: softmax of S_B(i)
//   slot B: matrix cores: O_B += V(i)^T P_B(i)^T, then S_B(i+1)^T = K(i+1) Q_B^T     vector ALUs: softmax of S_A(i+1)
// so every MFMA of one tile is issued between a few vector instructions of the other tile's softmax, and the two
// never wait for each other the way two separate waves on a SIMD do (those meet at the workgroup barrier of every
// block and compete for the issue port in whatever order the arbiter picks). The order is the source order: the
// MFMAs are asm statements (accumulators tied, O in AGPRs), and a full scheduling fence follows every position.
// K / V tiles sit in a ring of three LDS stages each, filled by buffer loads into LDS issued two blocks ahead (the
// barrier at the top of iteration i frees the stages of K(i) and V(i-1), which take K(i+3) and V(i+2)), so the wait
// at the top of a block is for copies that had a whole block to land. The copies are asm as well (the stage is picked
// at run time); this kernel does its own vmcnt waiting.
// Layouts (S^T = K Q^T with the K fragment first, P straight from the score registers, V through the transposing
// LDS read) are those of flash_fwd_kernel in flash_attn.hip.
#include <type_traits>
#include "flash_attn_tiles.h"

namespace hexmi {
namespace {

template <typename T> struct MfmaAsm;
template <> struct MfmaAsm<f16> {
  typedef f16x8 Frag;
  // first_v / acc_v: the score MFMAs. Their second operand (the Q fragment, fixed for a whole unit) is taken from an
  // AGPR, which keeps the 64 registers of the two tiles' Q fragments out of the arch VGPRs.
  // c = a b (srcC = 0): the first MFMA of a score chain
  static __device__ __forceinline__ void first_v(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void acc_v(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void acc_a(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct MfmaAsm<bf16> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ void first_v(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void acc_v(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "a"(b));
  }
  static __device__ __forceinline__ void acc_a(const Frag& a, const Frag& b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

// The output accumulators are not C++ values at all: tuple i (tile i/4, 32 columns i%4 of the head dimension) IS the
// AGPRs a[16i : 16i+15], named in the text of every statement that touches it and listed there as clobbered, so the
// compiler keeps its own values (the Q fragments, anything it parks in AGPRs) out of a0..a127 wherever such a value
// lives across one of these statements, which is everywhere in the key loop. (As a C++ value the accumulator has to
// pass through VGPRs in the rarely taken rescaling block, and the register allocator then places those copies on
// the path of every key block: 128 extra instructions per block for a wave that can issue one every four cycles.)
#define HEXMI_CLOB_0 "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15"
#define HEXMI_CLOB_1 "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31"
#define HEXMI_CLOB_2 "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47"
#define HEXMI_CLOB_3 "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63"
#define HEXMI_CLOB_4 "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79"
#define HEXMI_CLOB_5 "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95"
#define HEXMI_CLOB_6 "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111"
#define HEXMI_CLOB_7 "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127"
#define HEXMI_Z1(K) "v_accvgpr_write_b32 a[%0+" #K "], 0\n\t"
#define HEXMI_S1(K) "v_accvgpr_read_b32 %0, a[%2+" #K "]\n\tv_mul_f32 %0, %0, %1\n\ts_nop 0\n\tv_accvgpr_write_b32 a[%2+" #K "], %0\n\t"
#define HEXMI_X16(M) M(0) M(1) M(2) M(3) M(4) M(5) M(6) M(7) M(8) M(9) M(10) M(11) M(12) M(13) M(14) M(15)
template <int I> struct OAcc;
#define HEXMI_OACC(I, CLOB)                                                                                  \
  template <> struct OAcc<I> {                                                                               \
    static __device__ __forceinline__ void pv(const f16x8& a, const f16x8& b) {                              \
      asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]"                                      \
                   : : "v"(a), "v"(b), "n"(16 * I), "n"(16 * I + 15) : CLOB);                                \
    }                                                                                                        \
    static __device__ __forceinline__ void pv(const bf16x8& a, const bf16x8& b) {                            \
      asm volatile("v_mfma_f32_32x32x16_bf16 a[%2:%3], %0, %1, a[%2:%3]"                                     \
                   : : "v"(a), "v"(b), "n"(16 * I), "n"(16 * I + 15) : CLOB);                                \
    }                                                                                                        \
    static __device__ __forceinline__ void zero() { asm volatile(HEXMI_X16(HEXMI_Z1) : : "n"(16 * I) : CLOB); } \
    static __device__ __forceinline__ void scale(float alpha) {                                              \
      float tmp;                                                                                             \
      asm volatile(HEXMI_X16(HEXMI_S1) : "=&v"(tmp) : "v"(alpha), "n"(16 * I) : CLOB);                       \
    }                                                                                                        \
    template <int K> static __device__ __forceinline__ float get() {                                         \
      float x;                                                                                               \
      asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(16 * I + K));                              \
      return x;                                                                                              \
    }                                                                                                        \
  };
HEXMI_OACC(0, HEXMI_CLOB_0)
HEXMI_OACC(1, HEXMI_CLOB_1)
HEXMI_OACC(2, HEXMI_CLOB_2)
HEXMI_OACC(3, HEXMI_CLOB_3)
HEXMI_OACC(4, HEXMI_CLOB_4)
HEXMI_OACC(5, HEXMI_CLOB_5)
HEXMI_OACC(6, HEXMI_CLOB_6)
HEXMI_OACC(7, HEXMI_CLOB_7)
#undef HEXMI_OACC

constexpr int kPipeD = 128;
constexpr int kPipeRows = 256;                 // query rows per workgroup (4 waves x 64)
constexpr int kPipeTile = kBlockN * kPipeD;    // elements of one K or V stage
constexpr int kPipeStages = 3;
constexpr int kGroup = 4;                      // MFMAs per group: the fragments of a group are read in one burst,
constexpr int kAhead = 2 * kGroup;             // two groups (eight MFMAs) ahead of their use

// Maxima as asm: fmaxf() makes the compiler quiet signalling NaNs first (two extra instructions per pair), and a
// single wave can issue only one instruction every four cycles. A chain is one statement: between two asm statements
// that depend on each other the compiler leaves a wait state (it cannot tell that they are no transcendentals).
__device__ __forceinline__ float max8(float a, float b, float c, float d, float e, float f, float g, float h) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max_f32 %0, %0, %8"
      : "=&v"(r) : "v"(a), "v"(b), "v"(c), "v"(d), "v"(e), "v"(f), "v"(g), "v"(h));
  return r;
}
// max(a, b, c, d, e) where e arrives later than the others
__device__ __forceinline__ float max4(float a, float b, float c, float d) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3\n\tv_max_f32 %0, %0, %4" : "=&v"(r) : "v"(a), "v"(b), "v"(c), "v"(d));
  return r;
}

template <typename T, typename OutT, bool CAUSAL>
__global__ __launch_bounds__(256, 1)
void flash_fwd_pipe_kernel(const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
                           OutT* __restrict__ O, int ZH, int S, float scale_log2e) {
  typedef typename MfmaAsm<T>::Frag Frag;
  typedef __attribute__((address_space(3))) const Frag* LdsFrag;
  typedef __attribute__((address_space(3))) i16x4* LdsTr;
  typedef int i32x4v __attribute__((ext_vector_type(4)));
  constexpr int D = kPipeD, DS = D / 16, DT = D / 32, CPR = D / 8;
  constexpr int kStageBytes = kPipeTile * (int)sizeof(T);   // 16 KiB
  __shared__ __attribute__((aligned(16))) T k_ring[kPipeStages * kPipeTile];
  __shared__ __attribute__((aligned(16))) T v_ring[kPipeStages * kPipeTile];
  const unsigned k_lds = (unsigned)(uintptr_t)((__attribute__((address_space(3))) void*)(k_ring));
  const unsigned v_lds = (unsigned)(uintptr_t)((__attribute__((address_space(3))) void*)(v_ring));

  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int row32 = lane % 32, half = lane / 32;
  const int nqb = (S + kPipeRows - 1) / kPipeRows;

  // ---- per-lane constants of the tile layout (see swz_ktile / swz_vtile), in bytes ----
  // copies: instruction c (0..3) of a wave moves rows wave*4 + c*16 + lane/16 of a 64-row tile, one 16-byte chunk
  // per lane; the LDS side is linear in (c, wave, lane), the XOR swizzle is applied to the source column
  int cp_koff, cp_voff;                                     // byte offset of this lane's chunk inside a tile, c = 0
  {
    const int lin = wave * 64 + lane;
    const int r0 = lin / CPR, ch = lin % CPR;
    cp_koff = (r0 * D + ((ch ^ swz_ktile<D>(r0)) * 8)) * (int)sizeof(T);
    cp_voff = (r0 * D + ((ch ^ swz_vtile<D>(r0)) * 8)) * (int)sizeof(T);
  }
  const unsigned cp_lds = wave * 1024;                      // this wave's 1 KiB of each 4 KiB copy row group
  // K fragment (jt, ds): row jt*32 + row32, chunk (ds*2 + half) ^ (row & 15). ka[ds] is the LDS address in the
  // stage being read (moved from stage to stage by adding the distance), jt adds an immediate.
  unsigned ka[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ++ds)
    ka[ds] = k_lds + (row32 * CPR + ((ds * 2 + half) ^ (row32 & 15))) * 16;
  // V fragment (jt, hf, dt), two transposing reads pp = 0, 1: row jt*32 + hf*16 + 8*pp + 4*(g>>1) + (i16>>2),
  // column dt*32 + (g&1)*16 + (i16&3)*4
  unsigned va[DT];
  {
    const int g = lane / 16, i16 = lane % 16;
    const int vrow = 4 * (g >> 1) + (i16 >> 2);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const int col = dt * 32 + (g & 1) * 16 + (i16 & 3) * 4;
      va[dt] = v_lds + ((vrow * CPR + ((col / 8) ^ swz_vtile<D>(vrow))) * 8 + (col % 8)) * (int)sizeof(T);
    }
  }
  int ka_stage = 0, va_stage = 0;                           // the stages ka / va point into

  const int total = ZH * nqb;
  const bool by_xcd = ZH % 8 == 0 && gridDim.x % 8 == 0;
  const int P = by_xcd ? gridDim.x / 8 : gridDim.x;
  const int u_id = by_xcd ? blockIdx.x / 8 : blockIdx.x;
  const int list_len = by_xcd ? total / 8 : total;
  for (int it = 0; it * P < list_len; ++it) {
    const int unit = it * P + ((it & 1) ? P - 1 - u_id : u_id);
    if (unit >= list_len) continue;                         // workgroup-uniform
    int zh, qb;
    if (by_xcd) {
      zh = blockIdx.x % 8 + 8 * (unit / nqb);
      qb = nqb - 1 - unit % nqb;
    } else {
      zh = unit % ZH;
      qb = nqb - 1 - unit / ZH;
    }
    const int64_t base = (int64_t)zh * S * D;

    const int q0w = qb * kPipeRows + wave * 64;             // first query row of this wave (S % 64 == 0)
    const int key_end = CAUSAL ? ((qb + 1) * kPipeRows < S ? (qb + 1) * kPipeRows : S) : S;
    const int nb_wg = key_end / kBlockN;                    // key blocks of the workgroup
    int nb_w = 0;                                           // key blocks of this wave
    if (q0w < S) nb_w = CAUSAL ? q0w / kBlockN + 1 : nb_wg;

    // Q fragments of both tiles: lane = (row row32 of the tile, d = ds*16 + half*8 .. +8). They are the second operand
    // of every score MFMA and nothing else, so they are loaded straight into AGPRs (an asm load: a value the
    // compiler loads itself has its home in the arch VGPRs and is copied over before every use). The wait for them is
    // the vmcnt(0) behind the prologue's copies.
    Frag qf[2][DS];
    {
      const int qr = q0w < S ? q0w + row32 : row32;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
          const T* src = Q + base + (int64_t)(qr + 32 * t) * D + ds * 16 + half * 8;
          asm volatile("global_load_dwordx4 %0, %1, off" : "=a"(qf[t][ds]) : "v"(src) : "memory");
        }
    }
    OAcc<0>::zero(); OAcc<1>::zero(); OAcc<2>::zero(); OAcc<3>::zero();      // tile A
    OAcc<4>::zero(); OAcc<5>::zero(); OAcc<6>::zero(); OAcc<7>::zero();      // tile B
    f32x16 s[2][2];                                         // [tile][32-key half of the block]
    Frag pf[2][4];                                          // packed probabilities: [tile][jt*2 + hf]
    float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.0f, 0.0f}, neg_m[2] = {0.0f, 0.0f};

    // ---- global -> LDS copies: buffer loads into LDS, one descriptor per operand and unit, the key block and the
    //      row group c in the scalar offset, the LDS destination (stage, c, wave) in M0. M0 is not saved: nothing
    //      else in this kernel uses it.
    i32x4v k_rsrc, v_rsrc;
    {
      const uint64_t kb = reinterpret_cast<uint64_t>(K + base), vb = reinterpret_cast<uint64_t>(V + base);
      k_rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)kb);
      k_rsrc[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(kb >> 32) & 0xffffu));
      v_rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)vb);
      v_rsrc[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(vb >> 32) & 0xffffu));
      k_rsrc[2] = v_rsrc[2] = 0x7fffffff;
      k_rsrc[3] = v_rsrc[3] = 0x00020000;
    }
    // copy c of block blk_off (a byte offset: block * 16 KiB, clamped by the caller) into the stage at lds_stage
    auto copy_one = [&](const i32x4v& rsrc, int voff, unsigned lds_stage, int blk_off, int c) __attribute__((always_inline)) {
      const unsigned dst = lds_stage + cp_lds + c * 4096;
      const int soff = blk_off + c * 4096;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                   : : "s"(dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
    };
    auto blk_bytes = [&](int blk) __attribute__((always_inline)) {
      return (blk < nb_wg ? blk : nb_wg - 1) * kStageBytes;       // past the end: any valid block, the stage is free
    };

    // ---- LDS fragment reads ----
    auto read_k = [&](int jt, int ds) __attribute__((always_inline)) {
      return *(LdsFrag)(uintptr_t)(ka[ds] + jt * (32 * CPR * 16));
    };
    auto read_v = [&](int jt, int hf, int dt) __attribute__((always_inline)) {
      union { i16x4 h[2]; Frag f; } u;
#pragma unroll
      for (int pp = 0; pp < 2; ++pp)
        u.h[pp] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (LdsTr)(uintptr_t)(va[dt] + (jt * 32 + hf * 16 + 8 * pp) * (CPR * 16)));
      return u.f;
    };
    // dispatch on the tuple index (a constant once the loops are unrolled)
    auto o_pv = [&](int i, const Frag& a, const Frag& b) __attribute__((always_inline)) {
      switch (i) {
        case 0: OAcc<0>::pv(a, b); break;
        case 1: OAcc<1>::pv(a, b); break;
        case 2: OAcc<2>::pv(a, b); break;
        case 3: OAcc<3>::pv(a, b); break;
        case 4: OAcc<4>::pv(a, b); break;
        case 5: OAcc<5>::pv(a, b); break;
        case 6: OAcc<6>::pv(a, b); break;
        default: OAcc<7>::pv(a, b); break;
      }
    };
    // Fragment of MFMA position p of a slot: 0..15 are P V (jt, hf, dt), 16..31 are K Q^T (ds, jt)
    auto read_pos = [&](int p) __attribute__((always_inline)) {
      if (p < 16) return read_v(p / 8, (p / 4) % 2, p % 4);
      return read_k((p - 16) % 2, (p - 16) / 2);
    };
    auto mfma_pos = [&](int p, int t, const Frag& f) __attribute__((always_inline)) {
      if (p < 16) {
        o_pv(t * 4 + p % 4, f, pf[t][p / 4]);
      } else {
        const int ds = (p - 16) / 2, jt = (p - 16) % 2;
        if (ds == 0) MfmaAsm<T>::first_v(f, qf[t][ds], s[t][jt]);
        else MfmaAsm<T>::acc_v(f, qf[t][ds], s[t][jt]);
      }
    };
    // move ka / va to another stage
    auto ka_to = [&](int stage) __attribute__((always_inline)) {
      const int delta = (stage - ka_stage) * kStageBytes;
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) ka[ds] += delta;
      ka_stage = stage;
    };
    auto va_to = [&](int stage) __attribute__((always_inline)) {
      const int delta = (stage - va_stage) * kStageBytes;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) va[dt] += delta;
      va_stage = stage;
    };

    // ---- softmax of one tile, in pieces ----
    // The reference maximum m_i may trail the true running maximum by up to kRescaleLag (log2 units), so the output
    // accumulator and running sum are rescaled only when a row outgrows the lag (see flash_fwd_kernel).
    float part[4];
    float mblk;
    auto sm_max_piece = [&](int u, int q) __attribute__((always_inline)) {      // q = 0..3: 8 of the 32 scores
      const f32x16& sv = s[u][q / 2];
      const int b0 = (q % 2) * 8;
      part[q] = max8(sv[b0], sv[b0 + 1], sv[b0 + 2], sv[b0 + 3], sv[b0 + 4], sv[b0 + 5], sv[b0 + 6], sv[b0 + 7]);
    };
    auto sm_max_final = [&](int u) __attribute__((always_inline)) {
      float mx = max4(part[0], part[1], part[2], part[3]);
      const float ot = other_half(mx);
      asm("v_max_f32 %0, %1, %2" : "=v"(mx) : "v"(mx), "v"(ot));
      mblk = mx * scale_log2e;
      asm volatile("" : "+v"(mblk));
    };
    // live: false in the one slot that runs on scores of a key block past the wave's last (the stream is the same
    // for every block; there the softmax must leave the tile's state alone)
    auto sm_rescale = [&](int u, bool live) __attribute__((always_inline)) {
      const bool grow = live && mblk > m_i[u] + kRescaleLag;
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(grow) != 0, 0)) {
        const float m_new = grow ? mblk : m_i[u];
        const float alpha = grow ? __builtin_amdgcn_exp2f(m_i[u] - m_new) : 1.0f;
        l_i[u] *= alpha;
        m_i[u] = m_new;
        if (u == 0) { OAcc<0>::scale(alpha); OAcc<1>::scale(alpha); OAcc<2>::scale(alpha); OAcc<3>::scale(alpha); }
        else { OAcc<4>::scale(alpha); OAcc<5>::scale(alpha); OAcc<6>::scale(alpha); OAcc<7>::scale(alpha); }
        neg_m[u] = m_i[u] == -INFINITY ? 0.0f : -m_i[u];
      }
    };
    float pe[8];
    auto sm_exp_piece = [&](int u, int g, int k) __attribute__((always_inline)) {   // group g = fragment, k = 0..5
      const f32x16& sv = s[u][g / 2];
      const int b0 = (g % 2) * 8;
      if (k < 4) {
        pe[2 * k] = __builtin_amdgcn_exp2f(fmaf(sv[b0 + 2 * k], scale_log2e, neg_m[u]));
        pe[2 * k + 1] = __builtin_amdgcn_exp2f(fmaf(sv[b0 + 2 * k + 1], scale_log2e, neg_m[u]));
        asm volatile("" : "+v"(pe[2 * k]), "+v"(pe[2 * k + 1]));
      } else if (k == 4) {
        pf[u][g] = MfmaT<T>::pack(pe);
      } else {
        l_i[u] = MfmaT<T>::sum8(pf[u][g], l_i[u]);
        asm volatile("" : "+v"(l_i[u]));
      }
    };
    // causal diagonal block: keys past the row are removed before the maximum
    auto sm_mask = [&](int u, int n0) __attribute__((always_inline)) {
      asm volatile("" ::: "memory");                        // not to be turned into 64 unconditional selects
      const int d = q0w + 32 * u + row32 - n0 - 4 * half;   // key index (without the lane part) must be <= d
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (jt * 32 + 8 * (r / 4) + r % 4 > d) s[u][jt][r] = -INFINITY;
    };
    auto sm_all = [&](int u) __attribute__((always_inline)) {
#pragma unroll
      for (int q = 0; q < 4; ++q) sm_max_piece(u, q);
      sm_max_final(u);
      sm_rescale(u, true);
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int k = 0; k < 6; ++k) sm_exp_piece(u, g, k);
    };

    // ---- one slot: the MFMAs of tile t (P V of its block i on the stage va points into, then K Q^T of its block
    //      i+1 on ka's stage, into its scores) with the softmax of tile u = 1 - t (live: see sm_rescale) between them.
    //      The fragments of a group of kGroup MFMAs are read one group ahead: fb holds the first group's on entry and
    //      receives the next slot's first group (P V; before_next moves va to that slot's stage) on exit.
    auto slot = [&](auto t_c, Frag* fb, bool live, auto&& copy_at, auto&& before_next) __attribute__((always_inline)) {
      constexpr int t = decltype(t_c)::value, u = 1 - t;
      constexpr int NP = 32;
      Frag fr[NP + kAhead];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) fr[i] = fb[i];
      const float l_keep = l_i[u];
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        if (p % kGroup == 0) {
          if (p + kAhead == NP) before_next();
#pragma unroll
          for (int i = 0; i < kGroup; ++i) fr[p + kAhead + i] = read_pos((p + kAhead + i) % NP);
          __builtin_amdgcn_sched_barrier(0);
        }
        mfma_pos(p, t, fr[p]);
        copy_at(p);
        if (p < 4) sm_max_piece(u, p);
        else if (p == 4) sm_max_final(u);
        else if (p >= 8) sm_exp_piece(u, (p - 8) / 6, (p - 8) % 6);
        __builtin_amdgcn_sched_barrier(0);
        if (p == 5) {
          sm_rescale(u, live);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      l_i[u] = live ? l_i[u] : l_keep;
#pragma unroll
      for (int i = 0; i < kAhead; ++i) fb[i] = fr[NP + i];
    };
    static_assert(kAhead <= 16, "the fragments carried into a slot are P V fragments");
    typedef std::integral_constant<int, 0> TileA;
    typedef std::integral_constant<int, 1> TileB;
    auto nothing = []() {};
    auto no_copies = [](int) {};

    // ---- prologue. Iteration i of the loop below works on V(i) and K(i+1): tile A's P V(i) and K(i+1) Q^T with
    //      tile B's softmax of block i between them, then tile B's with tile A's softmax of block i+1. Before it the
    //      wave needs S_B(0) and P_A(0). Block b lives in stage b % 3. The top of iteration i waits for K(i+2) and
    //      V(i+1) (issued during iteration i-1; iteration i itself reads K(i+1) and V(i), and at its end the first
    //      fragments of V(i+1)), then issues K(i+3) and V(i+2) into the stages of K(i) and V(i-1).
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      copy_one(k_rsrc, cp_koff, k_lds, blk_bytes(0), c);
      copy_one(k_rsrc, cp_koff, k_lds + kStageBytes, blk_bytes(1), c);
      copy_one(v_rsrc, cp_voff, v_lds, blk_bytes(0), c);
      copy_one(k_rsrc, cp_koff, k_lds + 2 * kStageBytes, blk_bytes(2), c);
      copy_one(v_rsrc, cp_voff, v_lds + kStageBytes, blk_bytes(1), c);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    Frag fb[kAhead];
    ka_to(0);
    va_to(0);
    if (nb_w > 0) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ds = 0; ds < DS; ++ds)
#pragma unroll
          for (int jt = 0; jt < 2; ++jt) {
            const Frag kf = read_k(jt, ds);
            if (ds == 0) MfmaAsm<T>::first_v(kf, qf[t][ds], s[t][jt]);
            else MfmaAsm<T>::acc_v(kf, qf[t][ds], s[t][jt]);
          }
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");    // the scores are read next and the MFMAs are asm
      if (CAUSAL && nb_w == 1) sm_mask(0, 0);
      sm_all(0);
#pragma unroll
      for (int i = 0; i < kAhead; ++i) fb[i] = read_pos(i);
    }
    __builtin_amdgcn_sched_barrier(0);

    int st_v = 0, st_k = 1, st_v2 = 2, st_k3 = 0;           // stages of V(i), K(i+1), and of the copies V(i+2), K(i+3)
    for (int i = 0; i < nb_wg; ++i) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // this wave's share of K(i+2), V(i+1)
      __builtin_amdgcn_s_barrier();                         // everyone's; and every wave is done with K(i), V(i-1)
      const int n0 = i * kBlockN;
      const unsigned k_dst = k_lds + st_k3 * kStageBytes, v_dst = v_lds + st_v2 * kStageBytes;
      const int k_blk = blk_bytes(i + 3), v_blk = blk_bytes(i + 2);
      auto copies = [&](int p) __attribute__((always_inline)) {           // one copy after each of the first 8 MFMAs
        if (p < 4) copy_one(k_rsrc, cp_koff, k_dst, k_blk, p);
        else if (p < 8) copy_one(v_rsrc, cp_voff, v_dst, v_blk, p - 4);
      };
      if (i < nb_w) {
        // The same stream for every block. The wave's last block (i == nb_w - 1) has no block i+1: its K Q^T MFMAs
        // run on whatever the K(i+1) stage holds (a real or a repeated block, finite numbers) and tile A's softmax of
        // those scores is not live. Causal: the wave's last block is its diagonal block and gets the mask first.
        ka_to(st_k);
        const int st_v1 = st_v == 2 ? 0 : st_v + 1;
        if (CAUSAL && i == nb_w - 1) sm_mask(1, n0);
        slot(TileA{}, fb, true, copies, nothing);
        if (CAUSAL && i + 2 == nb_w) {
          asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // S_A(i+1) comes from the asm MFMAs just issued
          sm_mask(0, n0 + kBlockN);
        }
        slot(TileB{}, fb, i + 1 < nb_w, no_copies, [&]() __attribute__((always_inline)) { va_to(st_v1); });
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) copy_one(k_rsrc, cp_koff, k_dst, k_blk, c);
#pragma unroll
        for (int c = 0; c < 4; ++c) copy_one(v_rsrc, cp_voff, v_dst, v_blk, c);
      }
      st_v = st_v == 2 ? 0 : st_v + 1;
      st_k = st_k == 2 ? 0 : st_k + 1;
      st_v2 = st_v2 == 2 ? 0 : st_v2 + 1;
      st_k3 = st_k3 == 2 ? 0 : st_k3 + 1;
    }
    // the MFMAs are asm: nothing tells the compiler that the accumulators are still in flight
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- epilogue: register r of tuple t*4 + dt is O[row][dt*32 + 8*(r/4) + 4*half + r%4] * l
    if (nb_w > 0) {
      auto store_tuple = [&](auto i_c, OutT* o_row, float inv_l) __attribute__((always_inline)) {
        constexpr int I = decltype(i_c)::value;
        typedef OAcc<I> A;
        constexpr int dt = I % 4;
        store4o<OutT>(o_row + dt * 32 + 0 + 4 * half, A::template get<0>() * inv_l, A::template get<1>() * inv_l,
                      A::template get<2>() * inv_l, A::template get<3>() * inv_l);
        store4o<OutT>(o_row + dt * 32 + 8 + 4 * half, A::template get<4>() * inv_l, A::template get<5>() * inv_l,
                      A::template get<6>() * inv_l, A::template get<7>() * inv_l);
        store4o<OutT>(o_row + dt * 32 + 16 + 4 * half, A::template get<8>() * inv_l, A::template get<9>() * inv_l,
                      A::template get<10>() * inv_l, A::template get<11>() * inv_l);
        store4o<OutT>(o_row + dt * 32 + 24 + 4 * half, A::template get<12>() * inv_l, A::template get<13>() * inv_l,
                      A::template get<14>() * inv_l, A::template get<15>() * inv_l);
      };
      {
        const float inv_l = 1.0f / (l_i[0] + other_half(l_i[0]));
        OutT* o_row = O + base + (int64_t)(q0w + row32) * D;
        store_tuple(std::integral_constant<int, 0>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 1>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 2>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 3>{}, o_row, inv_l);
      }
      {
        const float inv_l = 1.0f / (l_i[1] + other_half(l_i[1]));
        OutT* o_row = O + base + (int64_t)(q0w + 32 + row32) * D;
        store_tuple(std::integral_constant<int, 4>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 5>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 6>{}, o_row, inv_l);
        store_tuple(std::integral_constant<int, 7>{}, o_row, inv_l);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");        // trailing copies land before the next unit reuses the ring
    __syncthreads();
  }
}

}  // namespace

// Launches the pipelined kernel when the shape fits it (D = 128, S % 64 == 0, 16-bit types) and there are enough
// 256-row units to fill the chip; returns false otherwise.
bool flash_attn_pipe(const void* Q, const void* K, const void* V, void* O, int64_t ZH, int64_t S, int64_t D,
                     float scale_log2e, bool causal, int in_dtype, int out_dtype, hipStream_t st, int* status) {
  if (D != kPipeD || S % kBlockN != 0 || S < 2 * kBlockN) return false;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return false;
  const int64_t units = (S + kPipeRows - 1) / kPipeRows * ZH;
  if (units > 0x7fffffff || units < cus) return false;
  int64_t blocks = (int64_t)cus / 8 * 8;
  if (blocks == 0 || units < blocks) blocks = units;
#define HEXMI_PIPE(T, OutT)                                                                                          \
  do {                                                                                                               \
    if (causal)                                                                                                      \
      hipLaunchKernelGGL((flash_fwd_pipe_kernel<T, OutT, true>), dim3((unsigned)blocks), dim3(256), 0, st,          \
                         static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),              \
                         static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e);                                      \
    else                                                                                                             \
      hipLaunchKernelGGL((flash_fwd_pipe_kernel<T, OutT, false>), dim3((unsigned)blocks), dim3(256), 0, st,         \
                         static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),              \
                         static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e);                                      \
  } while (0)
  if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F16) HEXMI_PIPE(f16, f16);
  else if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F32) HEXMI_PIPE(f16, float);
  else if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_BF16) HEXMI_PIPE(bf16, bf16);
  else if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_F32) HEXMI_PIPE(bf16, float);
  else return false;
#undef HEXMI_PIPE
  *status = launch_status();
  return true;
}

}  // namespace hexmi
