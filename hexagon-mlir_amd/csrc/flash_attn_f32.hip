// Flash-attention forward for fp32 operands on the fp32 matrix cores (v_mfma_f32_32x32x2_f32): the dtype of the
// reference's own test (test/python/triton/test_flash_attention.py:171-173: torch.rand fp32 Q, K, V, [1,1,1024,64],
// scale 0.5). Same scheme as the 16-bit kernel of flash_attn.hip, nothing rounded below fp32:
//   a workgroup of 4 waves owns 128 query rows (32 per wave), keys walk in blocks of BN (64 for D = 64, 32 for
//   D = 128), K and V blocks are copied global -> LDS with buffer loads, double buffered;
//   S^T = K Q^T: a lane holds 16 scores per 32-key tile of ONE query row (row lane%32), Q stays in registers;
//   online softmax in fp32 with exp2 (scale*log2e folded in), the reference maximum may lag by kRescaleLagF32;
//   O^T += V^T P^T: the probabilities go from the score registers straight into the MFMA (score register r is k
//   slot r: keys 8*(r/4) + r%4 for lanes 0..31 and + 4 for lanes 32..63), V values are read from LDS one per lane.
// An MFMA of this shape takes 64 cycles, so a key block is 8192 matrix cycles per wave against about 500 of
// vector work: the kernel is matrix-bound without any software pipelining.
//
// LDS tiles are [BN keys][D] fp32 in 16-byte chunks: K is read by 32 keys at one chunk position (chunk ^ key%16),
// V by 32 consecutive d of two keys four apart (chunk ^ 8*((key/4)%2) puts the two half-waves on disjoint banks).
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr float kRescaleLagF32 = 8.0f;
typedef float f32x4a __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float other_half_f32(float v) {
  const unsigned u = __builtin_bit_cast(unsigned, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const unsigned lo = r[0], hi = r[1];
  return __builtin_bit_cast(float, (threadIdx.x & 32) ? lo : hi);
}

// PADDED: the head is head_dim < D wide (a multiple of 4): rows are head_dim floats apart in memory and the tiles
// carry zero columns from head_dim to D -- a copy lane whose chunk lies there issues nothing, its LDS positions (which
// no other lane writes) are zeroed once; the Q chunks there are zero registers, the output columns are not stored.
template <int D, int BN, bool CAUSAL, bool MASKED, bool PADDED = false>
__global__ __launch_bounds__(256, D == 64 ? 2 : 1)
void flash_fwd_f32_kernel(const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V,
                          float* __restrict__ O, int ZH, int S, int Skv, float scale_log2e,
                          const float* __restrict__ Mk, float mask_factor, int head_dim = D) {
  const int dh = PADDED ? head_dim : D;             // floats between rows in memory
  constexpr int NT = BN / 32;                       // 32-key score tiles per key block
  constexpr int CPR = D / 4;                        // 16-byte chunks per row
  constexpr int DT = D / 32;                        // 32-wide output tiles over the head dimension
  constexpr int DQ = D / 8;                         // 16-byte chunks of Q per lane (one per 8 head dimensions)
  constexpr int NI = BN * CPR / 64 / 4;             // copy instructions per wave and tile
  constexpr int RPI = 64 / CPR;                     // rows per copy instruction
  __shared__ __attribute__((aligned(16))) float k_s0[BN * D];
  __shared__ __attribute__((aligned(16))) float k_s1[BN * D];
  __shared__ __attribute__((aligned(16))) float v_s0[BN * D];
  __shared__ __attribute__((aligned(16))) float v_s1[BN * D];

  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int nqb = (S + 127) / 128;
  const int zh = blockIdx.x % ZH;
  const int qb = nqb - 1 - blockIdx.x / ZH;         // longest (last) query blocks first
  const float* q_g = Q + (int64_t)zh * S * dh;
  const float* k_g = K + (int64_t)zh * Skv * dh;
  const float* v_g = V + (int64_t)zh * Skv * dh;
  const int q0 = qb * 128 + wave * 32;
  const int r32 = lane % 32, kh = lane / 32;
  const int qrow = q0 + r32;
  const int qr = qrow < S ? qrow : S - 1;

  // Q: chunk 2*dq + kh of the row: head dimensions 8*dq + 4*kh + e, the k slots of MFMA (dq, e)
  f32x4a qf[DQ];
#pragma unroll
  for (int dq = 0; dq < DQ; ++dq) {
    if (!PADDED || (2 * dq + kh) * 4 < dh) qf[dq] = *reinterpret_cast<const f32x4a*>(q_g + (int64_t)qr * dh + (2 * dq + kh) * 4);
    else qf[dq] = f32x4a{0.0f, 0.0f, 0.0f, 0.0f};
  }

  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.0f;
  float m_i = -INFINITY, l_i = 0.0f, neg_m = 0.0f;

  const int key_end = CAUSAL ? ((qb + 1) * 128 < S ? (qb + 1) * 128 : S) : Skv;
  const int n_steps = (key_end + BN - 1) / BN;

  // ---- K / V tile copies
  int row_c[NI], kcol[NI], vcol[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int inst = j * 4 + wave;
    row_c[j] = inst * RPI + lane / CPR;
    const int pc = lane % CPR;
    kcol[j] = (pc ^ (row_c[j] & 15)) * 4;
    vcol[j] = (pc ^ (((row_c[j] >> 2) & 1) << 3)) * 4;
  }
  if constexpr (PADDED) {
    // the zero columns of both stages, once (the first barrier of the key loop lies before the first fragment read)
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const f32x4a z = {0.0f, 0.0f, 0.0f, 0.0f};
      if (kcol[j] >= dh) {
        *reinterpret_cast<f32x4a*>(k_s0 + (j * 4 + wave) * 256 + lane * 4) = z;
        *reinterpret_cast<f32x4a*>(k_s1 + (j * 4 + wave) * 256 + lane * 4) = z;
      }
      if (vcol[j] >= dh) {
        *reinterpret_cast<f32x4a*>(v_s0 + (j * 4 + wave) * 256 + lane * 4) = z;
        *reinterpret_cast<f32x4a*>(v_s1 + (j * 4 + wave) * 256 + lane * 4) = z;
      }
    }
  }
  auto load_kv = [&](int step, float* k_dst, float* v_dst) __attribute__((always_inline)) {
    const char* kb = reinterpret_cast<const char*>(k_g);
    const char* vb = reinterpret_cast<const char*>(v_g);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      int key = step * BN + row_c[j];
      key = key < Skv ? key : Skv - 1;                // rows past the end repeat the last key (masked below)
      if (!PADDED || kcol[j] < dh) copy_to_lds(kb, (key * dh + kcol[j]) * (int)sizeof(float), k_dst + (j * 4 + wave) * 256);
      if (!PADDED || vcol[j] < dh) copy_to_lds(vb, (key * dh + vcol[j]) * (int)sizeof(float), v_dst + (j * 4 + wave) * 256);
    }
  };

  const float* mask_row = nullptr;
  if constexpr (MASKED) mask_row = Mk + ((int64_t)zh * S + qr) * Skv;

  auto process = [&](int step, const float* ks, const float* vs) __attribute__((always_inline)) {
    const int n0 = step * BN;
    if (CAUSAL && n0 > q0 + 31) return;               // wholly past this wave's rows (wave-uniform)
    f32x4a mk[NT][4];
    if constexpr (MASKED) {
#pragma unroll
      for (int jt = 0; jt < NT; ++jt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          int key = n0 + jt * 32 + 8 * g4 + 4 * kh;
          key = key + 4 <= Skv ? key : Skv - 4;       // past the end: any valid run, those scores are dropped
          mk[jt][g4] = *reinterpret_cast<const f32x4a*>(mask_row + key);
        }
    }
    // ---- scores: two accumulators per tile, so a chain never waits for its own previous MFMA (one when the mask
    //      values already hold 16 registers per tile)
    constexpr bool kDual = !MASKED;
    f32x16 s[NT], s2[kDual ? NT : 1];
#pragma unroll
    for (int jt = 0; jt < NT; ++jt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[jt][r] = 0.0f;
        if (kDual) s2[jt][r] = 0.0f;
      }
#pragma unroll
    for (int dq = 0; dq < DQ; ++dq) {
#pragma unroll
      for (int jt = 0; jt < NT; ++jt) {
        const int row = jt * 32 + r32;
        const f32x4a kf = *reinterpret_cast<const f32x4a*>(ks + row * D + (((2 * dq + kh) ^ (row & 15)) * 4));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (!kDual || e % 2 == 0) s[jt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[dq][e], s[jt], 0, 0, 0);
          else s2[jt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[dq][e], s2[jt], 0, 0, 0);
        }
      }
    }
    if constexpr (kDual) {
#pragma unroll
      for (int jt = 0; jt < NT; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[jt][r] += s2[jt][r];
    }
    if constexpr (MASKED) {
      // softmax(scale*s + mask) = softmax(scale * (s + mask/scale))
#pragma unroll
      for (int jt = 0; jt < NT; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[jt][r] = fmaf(mk[jt][r / 4][r % 4], mask_factor, s[jt][r]);
    }
    const bool need_mask = (CAUSAL && n0 + BN - 1 > q0) || (n0 + BN > Skv);
    if (need_mask) {
#pragma unroll
      for (int jt = 0; jt < NT; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = n0 + jt * 32 + 8 * (r / 4) + 4 * kh + r % 4;
          if ((CAUSAL && key > qrow) || key >= Skv) s[jt][r] = -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < NT; ++jt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[jt][r]);
    mx = fmaxf(mx, other_half_f32(mx));
    const float m_blk = mx * scale_log2e;
    const bool grow = m_blk > m_i + kRescaleLagF32;
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float m_new = grow ? m_blk : m_i;
      const float alpha = grow ? __builtin_amdgcn_exp2f(m_i - m_new) : 1.0f;
      l_i *= alpha;
      m_i = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
      neg_m = m_i == -INFINITY ? 0.0f : -m_i;       // a row with every key masked so far: exp2(-inf) = 0, not NaN
    }
    // ---- O^T += V^T P^T: score register r of a lane is k slot r
#pragma unroll
    for (int jt = 0; jt < NT; ++jt) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = __builtin_amdgcn_exp2f(fmaf(s[jt][r], scale_log2e, neg_m));
        l_i += p[r];
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = jt * 32 + 8 * (r / 4) + 4 * kh + r % 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const float vv = vs[key * D + ((dt * 32 + r32) ^ (kh << 5))];
          o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, p[r], o_acc[dt], 0, 0, 0);
        }
      }
    }
  };

  load_kv(0, k_s0, v_s0);
  int step = 0;
  for (; step + 1 < n_steps; step += 2) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    load_kv(step + 1, k_s1, v_s1);
    process(step, k_s0, v_s0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (step + 2 < n_steps) load_kv(step + 2, k_s0, v_s0);
    process(step + 1, k_s1, v_s1);
  }
  if (step < n_steps) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    process(step, k_s0, v_s0);
  }

  // ---- o_acc[dt][r] is O[qrow][dt*32 + 8*(r/4) + 4*kh + r%4] * l
  const float l_tot = l_i + other_half_f32(l_i);
  const float inv_l = 1.0f / l_tot;
  if (qrow < S) {
    float* o_row = O + ((int64_t)zh * S + qrow) * dh;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        if (!PADDED || dt * 32 + 8 * q4 + 4 * kh < dh)
          *reinterpret_cast<f32x4a*>(o_row + dt * 32 + 8 * q4 + 4 * kh) =
              f32x4a{o_acc[dt][q4 * 4 + 0] * inv_l, o_acc[dt][q4 * 4 + 1] * inv_l, o_acc[dt][q4 * 4 + 2] * inv_l,
                     o_acc[dt][q4 * 4 + 3] * inv_l};
  }
}

// Small grids (fewer 128-row workgroups than half the CUs, e.g. the reference test's single head of 1024 rows):
// a workgroup owns 32 query rows and its NW waves split the KEYS (wave w takes the w-th run of 32-key blocks), each
// with its own double-buffered K / V tiles, so a wave waits only for its own copies and the loop has no barrier.
// The NW partial results (m, l, O) of a row meet in LDS at the end. Four times (D = 64) or twice (D = 128) the
// workgroups of the row-split kernel, each wave with a quarter or half of the keys.
template <int D, int NW, bool CAUSAL>
__global__ __launch_bounds__(NW * 64, 1)
void flash_fwd_f32_split_kernel(const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V,
                                float* __restrict__ O, int ZH, int S, float scale_log2e) {
  constexpr int BN = 32, CPR = D / 4, DT = D / 32, DQ = D / 8;
  constexpr int TILE = BN * D;                      // floats per K or V tile
  constexpr int NI = BN * CPR / 64;                 // copy instructions per tile (one wave issues them all)
  constexpr int RPI = 64 / CPR;
  __shared__ __attribute__((aligned(16))) float stage[NW * 4 * TILE];   // [wave][buffer][K, V][TILE]: 128 KiB
  __shared__ float m_s[NW][32], l_s[NW][32];

  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int nqb = (S + 31) / 32;
  const int zh = blockIdx.x % ZH;
  const int qb = nqb - 1 - blockIdx.x / ZH;
  const float* q_g = Q + (int64_t)zh * S * D;
  const float* k_g = K + (int64_t)zh * S * D;
  const float* v_g = V + (int64_t)zh * S * D;
  const int q0 = qb * 32;
  const int r32 = lane % 32, kh = lane / 32;
  const int qrow = q0 + r32;
  const int qr = qrow < S ? qrow : S - 1;

  f32x4a qf[DQ];
#pragma unroll
  for (int dq = 0; dq < DQ; ++dq)
    qf[dq] = *reinterpret_cast<const f32x4a*>(q_g + (int64_t)qr * D + (2 * dq + kh) * 4);
  f32x16 o_acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.0f;
  float m_i = -INFINITY, l_i = 0.0f, neg_m = 0.0f;

  const int key_end = CAUSAL ? (q0 + 32 < S ? q0 + 32 : S) : S;
  const int n_steps = (key_end + BN - 1) / BN;
  const int per = (n_steps + NW - 1) / NW;
  const int s_begin = wave * per;
  const int s_end = s_begin + per < n_steps ? s_begin + per : n_steps;

  int row_c[NI], kcol[NI], vcol[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    row_c[j] = j * RPI + lane / CPR;
    const int pc = lane % CPR;
    kcol[j] = (pc ^ (row_c[j] & 15)) * 4;
    vcol[j] = (pc ^ (((row_c[j] >> 2) & 1) << 3)) * 4;
  }
  float* my = stage + wave * (4 * TILE);
  auto load_kv = [&](int step, float* k_dst, float* v_dst) __attribute__((always_inline)) {
    const char* kb = reinterpret_cast<const char*>(k_g);
    const char* vb = reinterpret_cast<const char*>(v_g);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      int key = step * BN + row_c[j];
      key = key < S ? key : S - 1;
      // wave-private tiles at a run-time base: copies the compiler does not see, waits of our own (below)
      copy_to_lds_asm(kb, (key * D + kcol[j]) * (int)sizeof(float), k_dst + j * 256);
      copy_to_lds_asm(vb, (key * D + vcol[j]) * (int)sizeof(float), v_dst + j * 256);
    }
  };
  auto process = [&](int step, const float* ks, const float* vs) __attribute__((always_inline)) {
    const int n0 = step * BN;
    f32x16 s, s2;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.0f; s2[r] = 0.0f; }
#pragma unroll
    for (int dq = 0; dq < DQ; ++dq) {
      const f32x4a kf = *reinterpret_cast<const f32x4a*>(ks + r32 * D + (((2 * dq + kh) ^ (r32 & 15)) * 4));
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (e % 2 == 0) s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[dq][e], s, 0, 0, 0);
        else s2 = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[dq][e], s2, 0, 0, 0);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] += s2[r];
    if ((CAUSAL && n0 + BN - 1 > q0) || n0 + BN > S) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = n0 + 8 * (r / 4) + 4 * kh + r % 4;
        if ((CAUSAL && key > qrow) || key >= S) s[r] = -INFINITY;
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[r]);
    mx = fmaxf(mx, other_half_f32(mx));
    const float m_blk = mx * scale_log2e;
    const bool grow = m_blk > m_i + kRescaleLagF32;
    if (__builtin_amdgcn_ballot_w64(grow) != 0) {
      const float m_new = grow ? m_blk : m_i;
      const float alpha = grow ? __builtin_amdgcn_exp2f(m_i - m_new) : 1.0f;
      l_i *= alpha;
      m_i = m_new;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
      neg_m = m_i == -INFINITY ? 0.0f : -m_i;
    }
    float p[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      p[r] = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2e, neg_m));
      l_i += p[r];
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = 8 * (r / 4) + 4 * kh + r % 4;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const float vv = vs[key * D + ((dt * 32 + r32) ^ (kh << 5))];
        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, p[r], o_acc[dt], 0, 0, 0);
      }
    }
  };

  float* k0 = my, *v0 = my + TILE, *k1 = my + 2 * TILE, *v1 = my + 3 * TILE;
  if (s_begin < s_end) load_kv(s_begin, k0, v0);
  // Q has landed before the loop: left to the compiler, its wait (down to vmcnt(0)) would sit at Q's first use
  // inside the loop and wait for the copies in flight as well, in every key block
  __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0) only
  int step = s_begin;
  for (; step + 1 < s_end; step += 2) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    load_kv(step + 1, k1, v1);
    process(step, k0, v0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (step + 2 < s_end) load_kv(step + 2, k0, v0);
    process(step + 1, k1, v1);
  }
  if (step < s_end) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    process(step, k0, v0);
  }

  // ---- the NW partial results of a row meet in LDS: this wave's O (still times its own l) over its first tile
  const float l_w = l_i + other_half_f32(l_i);
  if (kh == 0) {
    m_s[wave][r32] = m_i;
    l_s[wave][r32] = l_w;
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4)
      *reinterpret_cast<f32x4a*>(my + r32 * D + dt * 32 + 8 * q4 + 4 * kh) =
          f32x4a{o_acc[dt][q4 * 4 + 0], o_acc[dt][q4 * 4 + 1], o_acc[dt][q4 * 4 + 2], o_acc[dt][q4 * 4 + 3]};
  __syncthreads();
  {
    constexpr int TPR = NW * 2;                      // threads per row
    constexpr int FPT = D / TPR;                     // floats per thread
    const int q = threadIdx.x / TPR, part = threadIdx.x % TPR;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) m = fmaxf(m, m_s[w][q]);
    float sc[NW], l = 0.0f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      sc[w] = m_s[w][q] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_s[w][q] - m);
      l += l_s[w][q] * sc[w];
    }
    const float inv = 1.0f / l;
    if (q0 + q < S) {
      float* o_row = O + ((int64_t)zh * S + q0 + q) * D + part * FPT;
#pragma unroll
      for (int f = 0; f < FPT; f += 4) {
        f32x4a acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < NW; ++w) {
          const f32x4a v = *reinterpret_cast<const f32x4a*>(stage + w * (4 * TILE) + q * D + part * FPT + f);
          acc += v * sc[w];
        }
        *reinterpret_cast<f32x4a*>(o_row + f) = acc * inv;
      }
    }
  }
}

template <int D, int BN>
int launch(const float* Q, const float* K, const float* V, const float* mask, float* O, int64_t ZH, int64_t S,
           int64_t Skv, float scale_log2e, bool causal, hipStream_t st, int head_dim = D) {
  const int64_t blocks = (S + 127) / 128 * ZH;
  if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
  const float mask_factor = mask ? 1.44269504088896340736f / scale_log2e : 0.0f;      // mask / sm_scale
#define HEXMI_FA32(CZ, MK, PD) \
  hipLaunchKernelGGL((flash_fwd_f32_kernel<D, BN, CZ, MK, PD>), dim3((unsigned)blocks), dim3(256), 0, st, Q, K, V, O, \
                     (int)ZH, (int)S, (int)Skv, scale_log2e, mask, mask_factor, head_dim)
  if (head_dim < D) {
    if (mask) HEXMI_FA32(false, true, true);
    else if (causal) HEXMI_FA32(true, false, true);
    else HEXMI_FA32(false, false, true);
  } else {
    if (mask) HEXMI_FA32(false, true, false);
    else if (causal) HEXMI_FA32(true, false, false);
    else HEXMI_FA32(false, false, false);
  }
#undef HEXMI_FA32
  return launch_status();
}

}  // namespace

// True (and the kernel launched, status in *status) for head sizes up to 128 in multiples of 4 (64 and 128 are the
// kernels' own; narrower heads run them on padded tiles) with 16-byte aligned operands; a mask
// needs whole 16-byte runs (Skv % 4 == 0) and excludes causal.
bool flash_attn_f32_mfma(const float* Q, const float* K, const float* V, const float* mask, float* O, int64_t ZH,
                         int64_t S, int64_t Skv, int64_t D, float scale_log2e, bool causal, hipStream_t st,
                         int* status) {
  if (D < 4 || D > 128 || D % 4 != 0) return false;     // 64 and 128, or a narrower head on padded tiles
  // the row maximum is taken on the raw scores and scaled afterwards: right for a positive scale only
  if (!(scale_log2e > 0.0f)) return false;
  if (!aligned_to(Q, 16) || !aligned_to(K, 16) || !aligned_to(V, 16) || !aligned_to(O, 16)) return false;
  if (Skv * D * (int64_t)sizeof(float) >= 0x7fffffff) return false;     // 32-bit byte offsets inside a head
  if (causal && (mask || Skv != S)) return false;
  if (mask && (Skv % 4 != 0 || Skv < 4 || !aligned_to(mask, 16))) return false;
  const int cus = hexmi_num_cus();
  const int64_t row_split_groups = (S + 127) / 128 * ZH;
  if ((D == 64 || D == 128) && !mask && Skv == S && row_split_groups * 2 < (cus > 0 ? cus : 256) &&
      (S + 31) / 32 * ZH <= 0x7fffffff) {
    // too few 128-row workgroups for the chip: 32-row workgroups whose waves split the keys
    const unsigned blocks = (unsigned)((S + 31) / 32 * ZH);
#define HEXMI_FA32S(DD, NWW, CZ) \
  hipLaunchKernelGGL((flash_fwd_f32_split_kernel<DD, NWW, CZ>), dim3(blocks), dim3(NWW * 64), 0, st, Q, K, V, O, \
                     (int)ZH, (int)S, scale_log2e)
    if (D == 64) { if (causal) HEXMI_FA32S(64, 4, true); else HEXMI_FA32S(64, 4, false); }
    else { if (causal) HEXMI_FA32S(128, 2, true); else HEXMI_FA32S(128, 2, false); }
#undef HEXMI_FA32S
    *status = launch_status();
    return true;
  }
  *status = D <= 64 ? launch<64, 64>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, causal, st, (int)D)
                    : launch<128, 32>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, causal, st, (int)D);
  return true;
}

}  // namespace hexmi
