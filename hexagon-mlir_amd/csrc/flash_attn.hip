// Flash-attention forward: O = softmax(scale * Q K^T [+ causal mask]) V, [Z,H,S,D] contiguous.
//
// Matrix-core kernel (fp16 / bf16, D = 64 or 128): a workgroup of 4 waves owns 128 query rows (32 per wave) and
// walks the keys in blocks of 64. K and V blocks are copied global -> LDS with buffer loads (copy_to_lds), double
// buffered. Per key block and wave:
//   S^T = K Q^T  with v_mfma_f32_32x32x16 (K fragment first): a lane then holds 32 scores of ONE query row
//                (row = lane%32), so row max / row sum are in-lane reductions plus one exchange with lane^32;
//   online softmax in fp32 with exp2 and scale*log2(e) folded in (running max m, running sum l);
//   O^T += V^T P^T: the probabilities go straight from the score registers to the MFMA operand (the k-slot to
//                key assignment of an MFMA is free, so it is chosen to match the score register layout) and the
//                V fragment comes from LDS through the transposing read ds_read_b64_tr_b16.
// Causal: key blocks past the diagonal are skipped, the diagonal blocks are masked element-wise, and workgroups
// are numbered so the longest (last) query blocks start first.
//
// Other 16-bit head sizes in multiples of 8: below 128 on tiles padded with zero columns (PADDED), above 128 up to
// 256 as two 128-wide halves of the head (WIDE).
//
// fp32 inputs with head size 64 or 128 run the fp32 matrix-core kernels of flash_attn_f32.hip; other head sizes and
// unaligned operands take the plain one-wave-per-query-row kernel below.
#include <algorithm>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "flash_attn_tiles.h"

namespace hexmi {
namespace {

// global -> LDS copy of the additive-mask tile of one wave: [32 query rows][64 keys], 128 bytes per row, four
// wave-wide instructions of 8 rows each. A lane later reads 8-byte runs of its own row (lane%32), so the 16-byte
// chunks of a row are XOR swizzled by row/2: the 32 rows of a read then cover every bank twice, the minimum for
// 512 bytes. Keys past the end of the sequence are clamped to the last chunk (their scores are dropped anyway),
// rows past the last query to the last query.
template <typename T>
struct MaskTileLoader {
  int rowoff[4];                                            // element offset of this lane's row from the first row
  int col0;                                                 // first key of this lane's chunk inside the tile, j = 0
  __device__ __forceinline__ void init(int wave, int lane, int rows_left, int Skv) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      int r = wave * 32 + j * 8 + lane / 8;                 // row j*8 + lane/8 of the tile
      r = r < rows_left ? r : rows_left - 1;
      rowoff[j] = r * Skv;
    }
    col0 = ((lane % 8) ^ ((lane / 16) & 7)) * 8;            // swizzle (row/2)%8 = (lane/16 + 4*(j%2)) % 8
  }
  // mask_wg: the mask row of the workgroup's first query; lds: this wave's [32][64] tile of the stage
  __device__ __forceinline__ void issue_one(int j, const T* __restrict__ mask_wg, int key0, int Skv, T* lds) const {
    const char* base = reinterpret_cast<const char*>(mask_wg);
    int key = key0 + (col0 ^ ((j & 1) * 32));
    key = key + 8 <= Skv ? key : Skv - 8;
    copy_to_lds<T, 2>(base, (rowoff[j] + key) * (int)sizeof(T), lds + j * 512);      // the mask is read once
  }
  __device__ __forceinline__ void issue(const T* __restrict__ mask_wg, int key0, int Skv, T* lds) const {
#pragma unroll
    for (int j = 0; j < 4; ++j) issue_one(j, mask_wg, key0, Skv, lds);
  }
};

// GENERAL: the number of keys (Skv) may differ from the number of queries (S) and an additive mask
// [ZH, S, Skv] (same dtype as Q; may be null) is added to the scaled scores before the softmax, as
// tm_tensor.attention does (qcom_hexagon_backend/lib/Transforms/LowerTmTensor.cpp:157-160); with a mask Skv % 4 == 0.
// NW waves per workgroup (4 or 8), 32 query rows each: every K / V tile copied into LDS serves NW*32 query rows.
// Eight waves halve the L2 -> LDS copy traffic (each query block streams the whole K and V of its head), worth
// 1-9 % from 2048 keys on; short sequences and small grids prefer the larger number of 128-row workgroups. (Measured on random
// data the kernel is held back by the power limit more than by any stall: all-zero inputs run 30 % faster through
// the same instructions and the same memory traffic, as the dense GEMM also shows.)
// MASK_LDS (GENERAL, 8 waves, a mask with Skv % 8 == 0): the mask tiles are copied global -> LDS one key block ahead
// like K and V (no registers, whole 128-byte rows), instead of being loaded into registers in 8-byte runs at the
// top of the block that uses them.
// PADDED: the head is head_dim < D wide (a multiple of 8): Q, K, V and O rows are head_dim elements apart, the tiles
// carry zero columns from head_dim to D (they add nothing to Q K^T; the output columns there are not stored).
// WIDE (with PADDED, D = 128, four waves): a head of 128 < head_dim <= 256 columns as two 128-wide halves. The
// scores are the sum over both halves' K tiles, the output two sets of accumulators, the second half's tiles padded
// like a narrow head's; twice the LDS and about 100 registers more, so one workgroup per CU.
template <typename T, typename OutT, int D, bool CAUSAL, bool GENERAL = false, int NW = 4, bool MASK_LDS = false,
          bool PADDED = false, bool WIDE = false>
__global__ __launch_bounds__(NW * 64, NW == 4 && !WIDE ? (D == 64 && !GENERAL ? 3 : 2) : 1)
void flash_fwd_kernel(const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
                      OutT* __restrict__ O, int ZH, int S, float scale_log2e, const T* __restrict__ Mk = nullptr,
                      int Skv_arg = 0, float mask_factor = 0.0f, int group_heads = 0, int head_dim = D) {
  static_assert(!(CAUSAL && GENERAL), "the causal kernel has as many keys as queries and no mask");
  static_assert(!WIDE || (PADDED && D == 128 && NW == 4 && !GENERAL), "two halves of 128 columns, four waves, no mask");
  const int dh = PADDED ? head_dim : D;                 // elements between rows in memory
  static_assert(!MASK_LDS || (GENERAL && NW == 8), "staged mask tiles: general kernel, 8 waves");
  const int Skv = GENERAL ? Skv_arg : S;
  typedef typename MfmaT<T>::Frag Frag;
  constexpr int DS = D / 16;                        // 16-wide steps over the head dimension
  constexpr int DT = D / 32;                        // 32-wide output tiles over the head dimension
  constexpr int CPR = D / 8;
  __shared__ __attribute__((aligned(16))) T k_lds0[kBlockN * D];
  __shared__ __attribute__((aligned(16))) T k_lds1[kBlockN * D];
  __shared__ __attribute__((aligned(16))) T v_lds0[kBlockN * D];
  __shared__ __attribute__((aligned(16))) T v_lds1[kBlockN * D];
  // WIDE: the tiles of columns 128 .. 255
  __shared__ __attribute__((aligned(16))) T kb_lds0[WIDE ? kBlockN * D : 8];
  __shared__ __attribute__((aligned(16))) T kb_lds1[WIDE ? kBlockN * D : 8];
  __shared__ __attribute__((aligned(16))) T vb_lds0[WIDE ? kBlockN * D : 8];
  __shared__ __attribute__((aligned(16))) T vb_lds1[WIDE ? kBlockN * D : 8];
  __shared__ __attribute__((aligned(16))) T m_lds0[MASK_LDS ? NW * 32 * kBlockN : 8];
  __shared__ __attribute__((aligned(16))) T m_lds1[MASK_LDS ? NW * 32 * kBlockN : 8];

  constexpr int kBlockM = NW * 32;                  // query rows per workgroup
  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int nqb = (S + kBlockM - 1) / kBlockM;
  if constexpr (PADDED) {
    // the zero columns of both stages of K and V, once: no copy ever writes there (the first barrier of the key loop
    // lies between these writes and the first fragment read)
    KvTileLoader<T, D, false, NW, true> kz;
    KvTileLoader<T, D, true, NW, true> vz;
    kz.init(wave, lane, dh, WIDE ? dh - D : dh);
    vz.init(wave, lane, dh, WIDE ? dh - D : dh);
    kz.zero_padding(WIDE ? kb_lds0 : k_lds0, lane);
    kz.zero_padding(WIDE ? kb_lds1 : k_lds1, lane);
    vz.zero_padding(WIDE ? vb_lds0 : v_lds0, lane);
    vz.zero_padding(WIDE ? vb_lds1 : v_lds1, lane);
  }
  // Persistent workgroups: the grid is at most what the chip holds at once, and a workgroup walks several (head,
  // query block) units, which takes the per-unit launch cost and the idle tail out of short causal units.
  // Workgroup ids are dealt round-robin to the 8 XCDs (one L2 each): every XCD gets a list of whole heads, longest
  // query blocks first, and its workgroups take the list in snake order (unit it*P + u, then it*P + P-1-u, ...),
  // so a workgroup's long and short units alternate and the head in progress stays in the XCD's L2.
  // group_heads = G > 0 (causal, chosen by the host, see plan_causal_groups): the snake pairs a workgroup's long
  // unit of one pass with a short one of the next only when a pass is whole heads, or a head whole passes: 16 query
  // blocks on 32 workgroups per XCD are, 15 or 62 are not, and the causal kernel then ran 20-40 % below its rate at
  // the next power of two (S = 15872: 763 TFLOP/s against 1139 at 16384). With G the XCD's heads are taken G at a
  // time; a group's units are listed longest first across its heads (slot j: head j % G, query block
  // nqb - 1 - j / G) and padded with empty slots at the short end to whole passes. G = 2 at 16 blocks is the list
  // described above; 15 blocks run as 32 slots of which two are empty, 62 blocks as 64 of which two are.
  const int total = ZH * nqb;
  const bool by_xcd = ZH % 8 == 0 && gridDim.x % 8 == 0;
  const int P = by_xcd ? gridDim.x / 8 : gridDim.x;             // workgroups sharing one list
  const int u = by_xcd ? blockIdx.x / 8 : blockIdx.x;
  const int G = by_xcd ? group_heads : 0;
  const int heads = ZH / 8;                                     // of an XCD's list
  const int gs = G > 0 ? (G * nqb + P - 1) / P * P : 0;         // slots of a full group
  const int full = G > 0 ? heads / G : 0, rem = G > 0 ? heads % G : 0;
  const int list_len = G > 0 ? full * gs + (rem * nqb + P - 1) / P * P : (by_xcd ? total / 8 : total);
  for (int it = 0; it * P < list_len; ++it) {
    const int unit = it * P + ((it & 1) ? P - 1 - u : u);
    if (unit >= list_len) continue;                             // workgroup-uniform, like the one below
    int zh, qb;
    if (G > 0) {
      const int grp = unit < full * gs ? unit / gs : full;
      const int j = unit - grp * gs, gh = grp < full ? G : rem;
      qb = nqb - 1 - j / gh;
      if (qb < 0) continue;                                     // padding
      zh = blockIdx.x % 8 + 8 * (grp * G + j % gh);
    } else if (by_xcd) {
      zh = blockIdx.x % 8 + 8 * (unit / nqb);
      qb = nqb - 1 - unit % nqb;
    } else {
      zh = unit % ZH;
      qb = nqb - 1 - unit / ZH;
    }
    const int64_t base = (int64_t)zh * S * dh;
    const int64_t kv_base = (int64_t)zh * Skv * dh;
    const T* q_g = Q + base;
    const T* k_g = K + kv_base;
    const T* v_g = V + kv_base;

    const int q0 = qb * kBlockM + wave * 32;           // first query row of this wave
    const int qrow = q0 + lane % 32;                    // the query row this lane's scores belong to
    const int half = lane / 32;

    // Q fragments stay in registers: lane = (row lane%32, d = ds*16 + half*8 .. +8)
    Frag qf[DS];
    {
      const int qr = qrow < S ? qrow : S - 1;
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        if (!PADDED || ds * 16 + half * 8 < dh) qf[ds] = *reinterpret_cast<const Frag*>(q_g + (int64_t)qr * dh + ds * 16 + half * 8);
        else qf[ds] = Frag{};
      }
    }
    Frag qfb[WIDE ? DS : 1];                            // WIDE: columns 128 .. 255 of the query row
    if constexpr (WIDE) {
      const int qr = qrow < S ? qrow : S - 1;
#pragma unroll
      for (int ds = 0; ds < DS; ++ds) {
        if (D + ds * 16 + half * 8 < dh) qfb[ds] = *reinterpret_cast<const Frag*>(q_g + (int64_t)qr * dh + D + ds * 16 + half * 8);
        else qfb[ds] = Frag{};
      }
    }

    f32x16 o_acc[DT];
    f32x16 o_accb[WIDE ? DT : 1];                       // WIDE: output columns 128 .. 255
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        o_acc[dt][r] = 0.0f;
        if constexpr (WIDE) o_accb[dt][r] = 0.0f;
      }
    float m_i = -INFINITY;                              // running max (already multiplied by scale*log2e)
    float l_i = 0.0f;                                   // this lane's share of the running sum

    const int key_end = CAUSAL ? ((qb + 1) * kBlockM < S ? (qb + 1) * kBlockM : S) : Skv;
    const int n_steps = (key_end + kBlockN - 1) / kBlockN;

    KvTileLoader<T, D, false, NW, PADDED> k_loader;
    KvTileLoader<T, D, true, NW, PADDED> v_loader;
    k_loader.init(wave, lane, dh, dh);
    v_loader.init(wave, lane, dh, dh);
    KvTileLoader<T, D, false, NW, PADDED> kb_loader;   // WIDE: the second halves, from 128 columns into the rows
    KvTileLoader<T, D, true, NW, PADDED> vb_loader;
    if constexpr (WIDE) {
      kb_loader.init(wave, lane, dh, dh - D);
      vb_loader.init(wave, lane, dh, dh - D);
    }
    MaskTileLoader<T> m_loader;
    const T* mask_wg = nullptr;
    if constexpr (MASK_LDS) {
      mask_wg = Mk + ((int64_t)zh * S + qb * kBlockM) * Skv;
      m_loader.init(wave, lane, S - qb * kBlockM, Skv);
    }
    auto load_kv = [&](int step, T* k_dst, T* v_dst, T* m_dst, T* kb_dst, T* vb_dst) __attribute__((always_inline)) {
      k_loader.issue(k_g, step * kBlockN, Skv, k_dst);
      v_loader.issue(v_g, step * kBlockN, Skv, v_dst);
      if constexpr (WIDE) {
        kb_loader.issue(k_g + D, step * kBlockN, Skv, kb_dst);
        vb_loader.issue(v_g + D, step * kBlockN, Skv, vb_dst);
      }
      if constexpr (MASK_LDS) m_loader.issue(mask_wg, step * kBlockN, Skv, m_dst + wave * (32 * kBlockN));
    };
    // The same copies one instruction at a time (c = 0 .. kCopies-1: K, then V, then the mask), for issuing
    // them between the score MFMAs of the block before. Whole tiles only: a ragged last tile is copied by load_kv.
    constexpr int kNI = KvTileLoader<T, D, false, NW>::NI;
    constexpr int kCopies = (WIDE ? 4 : 2) * kNI + (MASK_LDS ? 4 : 0);
    auto load_one = [&](int c, int step, T* k_dst, T* v_dst, T* m_dst, T* kb_dst, T* vb_dst) __attribute__((always_inline)) {
      if (c < kNI) k_loader.issue_one_whole(c, k_g, step * kBlockN, k_dst);
      else if (c < 2 * kNI) v_loader.issue_one_whole(c - kNI, v_g, step * kBlockN, v_dst);
      else if constexpr (WIDE) {
        if (c < 3 * kNI) kb_loader.issue_one_whole(c - 2 * kNI, k_g + D, step * kBlockN, kb_dst);
        else vb_loader.issue_one_whole(c - 3 * kNI, v_g + D, step * kBlockN, vb_dst);
      } else if constexpr (MASK_LDS) m_loader.issue_one(c - 2 * kNI, mask_wg, step * kBlockN, Skv, m_dst + wave * (32 * kBlockN));
    };

    // Online softmax of one 64-key block (two 32-key score tiles): mask, row max, (rare) rescale; the exponentials
    // follow per tile (exp_tile). The reference maximum m_i may lag the true running maximum by up to kRescaleLag
    // (log2 units): softmax is shift invariant, so exponentials up to 2^kRescaleLag are as exact as ones below 1,
    // and the output accumulator and running sum only need rescaling when a row outgrows the lag. The decision is
    // per row (lane); the wave-uniform ballot only skips the multiplications when no row of the wave needs them.
    // One decision per block (not per tile) leaves one branch between the score MFMAs and everything after them,
    // so the exponentials of the second tile can be scheduled under the P V MFMAs of the first.
    float neg_m = 0.0f;                                 // -(reference maximum) as the exponentials use it
    auto block_max = [&](int n0, bool need_mask, f32x16* s) __attribute__((always_inline)) {
      if (need_mask) {
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = n0 + jt * 32 + 8 * (r / 4) + 4 * half + r % 4;
            if ((CAUSAL && key > qrow) || key >= Skv) s[jt][r] = -INFINITY;
          }
      }
      float mx = -INFINITY, mx1 = -INFINITY;            // one chain per tile: three-operand maxima, no NaN quieting
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[0][r]);
#pragma unroll
      for (int r = 0; r < 16; ++r) mx1 = fmaxf(mx1, s[1][r]);
      mx = fmaxf(mx, mx1);
      mx = fmaxf(mx, other_half(mx));
      const float m_blk = mx * scale_log2e;
      const bool grow = m_blk > m_i + kRescaleLag;
      if (__builtin_amdgcn_ballot_w64(grow) != 0) {
        const float m_new = grow ? m_blk : m_i;
        const float alpha = grow ? __builtin_amdgcn_exp2f(m_i - m_new) : 1.0f;
        l_i *= alpha;
        m_i = m_new;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            o_acc[dt][r] *= alpha;
            if constexpr (WIDE) o_accb[dt][r] *= alpha;
          }
        // a row with every key masked so far keeps m_i = -inf and neg_m = 0: its scores are all -inf and give
        // exp2(-inf) = 0, not exp2(-inf + inf)
        neg_m = m_i == -INFINITY ? 0.0f : -m_i;
      }
    };
    // probabilities of one 32-key tile as the two MFMA operands pf[0], pf[1] (score registers 0..7 and 8..15 of
    // this lane), and their sum into l_i
    auto exp_tile = [&](const f32x16& s, Frag* pf) __attribute__((always_inline)) {
      float p[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) p[r] = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2e, neg_m));
      pf[0] = MfmaT<T>::pack(&p[0]);
      pf[1] = MfmaT<T>::pack(&p[8]);
      // the running sum takes the probabilities as rounded for the matrix cores (what P V actually multiplies),
      // two per instruction
      l_i = MfmaT<T>::sum8(pf[1], MfmaT<T>::sum8(pf[0], l_i));
    };
    // O^T += V^T P^T for one 32-key tile. MFMA k-slot (half h, e) <-> key jt*32 + hf*16 + 8*(e/4) + 4*h + e%4,
    // which is score register hf*8 + e of this lane, so the packed probabilities are used as they are. The V
    // fragments of a tile (read_v) do not depend on the scores: the first tile's are read before the softmax so
    // their LDS latency is spent under it.
    struct VFrags { Frag f[2][DT]; };
    auto read_v = [&](const T* v_src, int jt, VFrags& vf) __attribute__((always_inline)) {
      const int g = lane / 16, i16 = lane % 16;
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          union { i16x4 h[2]; Frag f; } u;
#pragma unroll
          for (int pp = 0; pp < 2; ++pp) {
            const int row = jt * 32 + hf * 16 + 8 * pp + 4 * (g >> 1) + (i16 >> 2);
            const int col = dt * 32 + (g & 1) * 16 + (i16 & 3) * 4;
            const int c = (col / 8) ^ swz_vtile<D>(row);
            const T* addr = v_src + (row * CPR + c) * 8 + (col % 8);
            u.h[pp] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(addr));
          }
          vf.f[hf][dt] = u.f;
        }
      }
    };
    auto pv_tile = [&](const VFrags& vf, const Frag* pf) __attribute__((always_inline)) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o_acc[dt] = MfmaT<T>::run(vf.f[hf][dt], pf[hf], o_acc[dt]);
    };
    auto pv_tile_b = [&](const VFrags& vf, const Frag* pf) __attribute__((always_inline)) {
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int dt = 0; dt < (WIDE ? DT : 1); ++dt) o_accb[dt] = MfmaT<T>::run(vf.f[hf][dt], pf[hf], o_accb[dt]);
    };

    // mask row of this lane's query (GENERAL with a mask only)
    const T* mask_row = nullptr;
    if constexpr (GENERAL && !MASK_LDS) {
      if (Mk) mask_row = Mk + ((int64_t)zh * S + (qrow < S ? qrow : S - 1)) * Skv;
    }

    // One key block. The global -> LDS copies of the next block (next >= 0, into the other stage) are issued a
    // few at a time between the score MFMAs: issued in one burst after the barrier, the 32 KiB of a block keep the
    // CU's vector memory pipe busy for about 500 cycles, during which every wave sits in its copy instructions
    // and the matrix cores have nothing queued.
    auto process = [&](int step, const T* k_src, const T* v_src, const T* m_src, int next, T* k_dst, T* v_dst,
                       T* m_dst, const T* kb_src, const T* vb_src, T* kb_dst, T* vb_dst) __attribute__((always_inline)) {
      const int n0 = step * kBlockN;
      // causal: a key block wholly past this wave's 32 rows contributes nothing (wave-uniform; the workgroup's
      // barriers are outside)
      const bool spread = next >= 0 && (next + 1) * kBlockN <= Skv && !(CAUSAL && n0 > q0 + 31);
      if (next >= 0 && !spread) load_kv(next, k_dst, v_dst, m_dst, kb_dst, vb_dst);
      if (CAUSAL && n0 > q0 + 31) return;
      // mask values of this lane's 32 scores: four runs of four consecutive keys per 32-key tile
      typedef T MaskRun __attribute__((ext_vector_type(4)));
      MaskRun mk[2][4];
      if constexpr (GENERAL && !MASK_LDS) {
        if (mask_row) {
#pragma unroll
          for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
              int key = n0 + jt * 32 + 8 * g4 + 4 * half;
              key = key + 4 <= Skv ? key : Skv - 4;          // past the end: any valid run, those scores are dropped
              mk[jt][g4] = *reinterpret_cast<const MaskRun*>(mask_row + key);
            }
        }
      }
      // ---- scores: s[jt][r] = Q[qrow] . K[n0 + jt*32 + 8*(r/4) + 4*half + r%4]. The MFMA chains of the two 32-key
      // tiles are interleaved (a chain alone waits for its own previous result) and their K fragments are read
      // kAhead steps ahead of use, so the LDS latency is paid once per block and not once per step.
      f32x16 s[2];
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[jt][r] = 0.0f;
      {
        constexpr int kAhead = GENERAL ? 2 : 3;      // the masked kernel holds its mask values too
        const int krow = lane % 32;
        auto read_k = [&](int jt, int ds) __attribute__((always_inline)) {
          const int row = jt * 32 + krow;
          const int c = (ds * 2 + half) ^ swz_ktile<D>(row);
          return *reinterpret_cast<const Frag*>(k_src + (row * CPR + c) * 8);
        };
        Frag kf[2][DS];
#pragma unroll
        for (int ds = 0; ds < kAhead && ds < DS; ++ds) {
          kf[0][ds] = read_k(0, ds);
          kf[1][ds] = read_k(1, ds);
        }
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
          if (ds + kAhead < DS) {
            kf[0][ds + kAhead] = read_k(0, ds + kAhead);
            kf[1][ds + kAhead] = read_k(1, ds + kAhead);
          }
          s[0] = MfmaT<T>::run(kf[0][ds], qf[ds], s[0]);
          s[1] = MfmaT<T>::run(kf[1][ds], qf[ds], s[1]);
          if (spread) {
#pragma unroll
            for (int c = 0; c < kCopies; ++c)
              if (c * DS / kCopies == ds) load_one(c, next, k_dst, v_dst, m_dst, kb_dst, vb_dst);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (WIDE) {                           // the second halves of Q and K add to the same scores
          auto read_kb = [&](int jt, int ds) __attribute__((always_inline)) {
            const int row = jt * 32 + krow;
            const int c = (ds * 2 + half) ^ swz_ktile<D>(row);
            return *reinterpret_cast<const Frag*>(kb_src + (row * CPR + c) * 8);
          };
#pragma unroll
          for (int ds = 0; ds < kAhead && ds < DS; ++ds) {
            kf[0][ds] = read_kb(0, ds);
            kf[1][ds] = read_kb(1, ds);
          }
#pragma unroll
          for (int ds = 0; ds < DS; ++ds) {
            if (ds + kAhead < DS) {
              kf[0][ds + kAhead] = read_kb(0, ds + kAhead);
              kf[1][ds + kAhead] = read_kb(1, ds + kAhead);
            }
            s[0] = MfmaT<T>::run(kf[0][ds], qfb[ds], s[0]);
            s[1] = MfmaT<T>::run(kf[1][ds], qfb[ds], s[1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      VFrags vf0, vf1;
      constexpr bool kEarlyV = !GENERAL;                // the masked kernel has no registers to spare for it
      if constexpr (kEarlyV) {
        read_v(v_src, 0, vf0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (MASK_LDS) {                         // staged mask tile: read after the score MFMAs are issued
        const int row = lane % 32;
        const T* m_row = m_src + wave * (32 * kBlockN) + row * kBlockN + half * 4;
#pragma unroll
        for (int jt = 0; jt < 2; ++jt)
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4)
            mk[jt][g4] = *reinterpret_cast<const MaskRun*>(m_row + ((jt * 4 + g4) ^ ((row >> 1) & 7)) * 8);
      }
      if constexpr (GENERAL) {
        if (MASK_LDS || mask_row) {
          // softmax(scale*s + mask) = softmax(scale * (s + mask/scale)): fold the mask into the raw scores
#pragma unroll
          for (int jt = 0; jt < 2; ++jt)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[jt][r] = fmaf(to_f32<T>(mk[jt][r / 4][r % 4]), mask_factor, s[jt][r]);
        }
      }
      const bool need_mask = (CAUSAL && n0 + kBlockN - 1 > q0) || (n0 + kBlockN > Skv);
      block_max(n0, need_mask, s);
      // The exponentials of tile 1 run on the vector ALUs while the matrix cores accumulate P V of tile 0.
      Frag pf[4];
      if constexpr (!kEarlyV) read_v(v_src, 0, vf0);
      read_v(v_src, 1, vf1);
      exp_tile(s[0], &pf[0]);
      pv_tile(vf0, &pf[0]);
      exp_tile(s[1], &pf[2]);
      pv_tile(vf1, &pf[2]);
      if constexpr (WIDE) {                             // the same probabilities on the second half of V
        read_v(vb_src, 0, vf0);
        read_v(vb_src, 1, vf1);
        pv_tile_b(vf0, &pf[0]);
        pv_tile_b(vf1, &pf[2]);
      }
    };

    load_kv(0, k_lds0, v_lds0, m_lds0, kb_lds0, vb_lds0);
    int step = 0;
    for (; step + 1 < n_steps; step += 2) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      process(step, k_lds0, v_lds0, m_lds0, step + 1, k_lds1, v_lds1, m_lds1, kb_lds0, vb_lds0, kb_lds1, vb_lds1);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      process(step + 1, k_lds1, v_lds1, m_lds1, step + 2 < n_steps ? step + 2 : -1, k_lds0, v_lds0, m_lds0, kb_lds1,
              vb_lds1, kb_lds0, vb_lds0);
    }
    if (step < n_steps) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      process(step, k_lds0, v_lds0, m_lds0, -1, k_lds1, v_lds1, m_lds1, kb_lds0, vb_lds0, kb_lds1, vb_lds1);
    }

    // ---- epilogue: o_acc[dt][r] is O[qrow][dt*32 + 8*(r/4) + 4*half + r%4] * l
    const float l_tot = l_i + other_half(l_i);
    const float inv_l = 1.0f / l_tot;
    if (qrow < S) {
      OutT* o_row = O + base + (int64_t)qrow * dh;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const int d = dt * 32 + 8 * q4 + 4 * half;
          if (!PADDED || d < dh)
            store4o<OutT>(o_row + d, o_acc[dt][q4 * 4 + 0] * inv_l, o_acc[dt][q4 * 4 + 1] * inv_l,
                          o_acc[dt][q4 * 4 + 2] * inv_l, o_acc[dt][q4 * 4 + 3] * inv_l);
          if constexpr (WIDE) {
            if (D + d < dh)
              store4o<OutT>(o_row + D + d, o_accb[dt][q4 * 4 + 0] * inv_l, o_accb[dt][q4 * 4 + 1] * inv_l,
                            o_accb[dt][q4 * 4 + 2] * inv_l, o_accb[dt][q4 * 4 + 3] * inv_l);
          }
        }
    }
    __syncthreads();                                            // the next unit's copies reuse both stages
  }
}

// fp32 (or any dtype / head size <= DMAX): one wave per query row; lanes take keys lane, lane+64, ...; each lane
// keeps its own (m, l, o[D]) and the 64 partial states are merged at the end.
template <typename T, typename OutT, int DMAX>
__global__ __launch_bounds__(256)
void flash_fwd_rowwise(const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V,
                       OutT* __restrict__ O, int64_t rows_total, int S, int D, float scale_log2e, int causal,
                       const T* __restrict__ Mk, int Skv) {
  __shared__ float q_s[4][DMAX];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;      // over ZH*S
  if (row >= rows_total) return;
  const int64_t zh = row / S;
  const int qi = (int)(row % S);
  const T* q = Q + row * D;
  const T* k = K + zh * Skv * D;
  const T* v = V + zh * Skv * D;
  const T* mrow = Mk ? Mk + row * Skv : nullptr;         // additive mask row [Skv] of this query
  for (int d = lane; d < D; d += kWave) q_s[wave][d] = to_f32<T>(q[d]);
  __builtin_amdgcn_wave_barrier();
  float o[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) o[d] = 0.0f;
  float m = -INFINITY, l = 0.0f;
  const int kend = causal ? qi + 1 : Skv;
  for (int j = lane; j < kend; j += kWave) {
    const T* kj = k + (int64_t)j * D;
    float sdot = 0.0f;
    for (int d = 0; d < D; ++d) sdot = fmaf(q_s[wave][d], to_f32<T>(kj[d]), sdot);
    float sv = sdot * scale_log2e;
    if (mrow) sv = fmaf(to_f32<T>(mrow[j]), 1.44269504088896340736f, sv);
    const float m_new = fmaxf(m, sv);
    if (m_new == -INFINITY) continue;                      // masked out so far: nothing to accumulate
    const float alpha = exp2f(m - m_new);
    const float p = exp2f(sv - m_new);
    l = l * alpha + p;
    const T* vj = v + (int64_t)j * D;
#pragma unroll
    for (int d = 0; d < DMAX; ++d)
      if (d < D) o[d] = o[d] * alpha + p * to_f32<T>(vj[d]);
    m = m_new;
  }
  const float m_all = wave_max(m);
  const float w = (m == -INFINITY) ? 0.0f : exp2f(m - m_all);
  const float l_all = wave_sum(l * w);
  const float inv = 1.0f / l_all;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) {
    if (d < D) {
      const float od = wave_sum(o[d] * w);
      if (lane == 0) O[row * D + d] = from_f32<OutT>(od * inv);
    }
  }
}

// Grid of the persistent kernel: what the chip holds at once (a multiple of 8 so every XCD gets the same number
// of workgroups), or one workgroup per unit when there are fewer units than that.
inline int64_t resident_grid(int64_t units, int per_cu) {
  const int cus = hexmi_num_cus();
  if (cus <= 0) return -1;
  const int64_t resident = (int64_t)cus * per_cu / 8 * 8;
  return units < resident || resident == 0 ? units : resident;
}

// Heads per group for the causal kernel's unit lists (0: the plain list of whole heads): the candidate whose
// busiest workgroup has the least to do, counted in key blocks plus two per unit, with the lists walked exactly as
// the kernel walks them; of equal candidates the largest group. Up to eight heads: more heads in flight per XCD
// than their keys and values fit its L2 cost nothing measurable ([4, 32, S, 128]: S = 3840 514 / 506 / 491 us with
// 2 / 4 / 8 heads, all equal in this count; S = 4096 567 / 574 / 552; S = 4352 842 / 644 / 632), balance decides.
inline int plan_causal_groups(int64_t ZH, int64_t nqb, int64_t grid) {
  if (ZH % 8 != 0 || grid % 8 != 0 || nqb > (1 << 20)) return 0;
  const int64_t P = grid / 8, heads = ZH / 8;
  if (heads * nqb <= P) return 0;                               // one unit per workgroup at most
  const int64_t gmax = heads < 8 ? heads : 8;
  // the answer depends on four integers: remembered, so that a launch does not pay for the walk
  static std::mutex mu;
  static std::map<std::tuple<int64_t, int64_t, int64_t, int64_t>, int> known;
  const auto key = std::make_tuple(ZH, nqb, grid, gmax);
  {
    std::lock_guard<std::mutex> lock(mu);
    const auto it = known.find(key);
    if (it != known.end()) return it->second;
  }
  std::vector<int64_t> load((size_t)P);
  int best = 0;
  int64_t best_span = -1;
  for (int G = 0; G <= (int)gmax; ++G) {
    std::fill(load.begin(), load.end(), 0);
    const int64_t gs = G > 0 ? (G * nqb + P - 1) / P * P : 0;
    const int64_t full = G > 0 ? heads / G : 0, rem = G > 0 ? heads % G : 0;
    const int64_t list_len = G > 0 ? full * gs + (rem * nqb + P - 1) / P * P : heads * nqb;
    for (int64_t it = 0; it * P < list_len; ++it)
      for (int64_t u = 0; u < P; ++u) {
        const int64_t unit = it * P + ((it & 1) ? P - 1 - u : u);
        if (unit >= list_len) continue;
        int64_t qb;
        if (G > 0) {
          const int64_t grp = unit < full * gs ? unit / gs : full;
          const int64_t j = unit - grp * gs, gh = grp < full ? G : rem;
          qb = nqb - 1 - j / gh;
          if (qb < 0) continue;
        } else {
          qb = nqb - 1 - unit % nqb;
        }
        load[(size_t)u] += qb + 2;
      }
    const int64_t span = *std::max_element(load.begin(), load.end());
    if (best_span < 0 || span <= best_span) {
      best_span = span;
      best = G;
    }
  }
  std::lock_guard<std::mutex> lock(mu);
  if (known.size() >= 1024) known.clear();                      // a caller with ever new shapes: start over
  known[key] = best;
  return best;
}

template <typename T, typename OutT, int D, bool CAUSAL, int NW>
int launch_mfma_nw(const void* Q, const void* K, const void* V, void* O, int64_t ZH, int64_t S, float scale_log2e,
                   hipStream_t st, int per_cu = NW == 4 ? 2 : 1) {
  const int64_t nqb = (S + NW * 32 - 1) / (NW * 32);
  const int64_t units = nqb * ZH;
  if (units > 0x7fffffff) return HEXMI_ENOTSUP;
  const int64_t blocks = resident_grid(units, per_cu);
  if (blocks <= 0) return HEXMI_ELAUNCH;
  const int groups = CAUSAL ? plan_causal_groups(ZH, nqb, blocks) : 0;
  hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, D, CAUSAL, false, NW>), dim3((unsigned)blocks), dim3(NW * 64), 0, st,
                     static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                     static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(nullptr), 0, 0.0f,
                     groups);
  return launch_status();
}

// A head of head_dim < D columns (a multiple of 8) on the kernel for D: 128-row workgroups, two per CU.
template <typename T, typename OutT, int D, bool CAUSAL>
int launch_mfma_padded(const void* Q, const void* K, const void* V, void* O, int64_t ZH, int64_t S, int head_dim,
                       float scale_log2e, hipStream_t st) {
  const int64_t nqb = (S + 127) / 128;
  const int64_t units = nqb * ZH;
  if (units > 0x7fffffff) return HEXMI_ENOTSUP;
  const int64_t blocks = resident_grid(units, 2);
  if (blocks <= 0) return HEXMI_ELAUNCH;
  const int groups = CAUSAL ? plan_causal_groups(ZH, nqb, blocks) : 0;
  hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, D, CAUSAL, false, 4, false, true>), dim3((unsigned)blocks), dim3(256), 0, st,
                     static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                     static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(nullptr), 0, 0.0f,
                     groups, head_dim);
  return launch_status();
}

// A head of 128 < head_dim <= 256 columns (a multiple of 8) as two halves on the kernel for 128: one 128-row
// workgroup per CU.
template <typename T, typename OutT, bool CAUSAL>
int launch_mfma_wide(const void* Q, const void* K, const void* V, void* O, int64_t ZH, int64_t S, int head_dim,
                     float scale_log2e, hipStream_t st) {
  const int64_t nqb = (S + 127) / 128;
  const int64_t units = nqb * ZH;
  if (units > 0x7fffffff) return HEXMI_ENOTSUP;
  const int64_t blocks = resident_grid(units, 1);
  if (blocks <= 0) return HEXMI_ELAUNCH;
  const int groups = CAUSAL ? plan_causal_groups(ZH, nqb, blocks) : 0;
  hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, 128, CAUSAL, false, 4, false, true, true>), dim3((unsigned)blocks), dim3(256), 0,
                     st, static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                     static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(nullptr), 0, 0.0f,
                     groups, head_dim);
  return launch_status();
}

template <typename T, typename OutT, int D>
int launch_mfma(const void* Q, const void* K, const void* V, void* O, int64_t ZH, int64_t S, float scale_log2e,
                bool causal, hipStream_t st) {
  // 256-row workgroups halve the L2 -> LDS copy traffic (1-9 % faster from 2048 keys on), if there are enough of
  // them to fill the chip; smaller problems keep the larger number of 128-row workgroups
  const bool wide = S >= kWideMinS && ZH * ((S + 255) / 256) >= hexmi_num_cus();
  // D = 64 leaves room for three 128-row workgroups per CU (144-154 registers): 6-9 % faster than the 256-row ones
  // between 2048 and 4095 keys when every workgroup still gets two units or more; fewer units balance better two per CU
  const bool three = D == 64 && S >= kWideMinS && S < 4096 && ZH * ((S + 127) / 128) >= 6 * (int64_t)hexmi_num_cus();
  if (three) {
    if (causal) return launch_mfma_nw<T, OutT, D, true, 4>(Q, K, V, O, ZH, S, scale_log2e, st, 3);
    return launch_mfma_nw<T, OutT, D, false, 4>(Q, K, V, O, ZH, S, scale_log2e, st, 3);
  }
  if (causal) {
    if (wide) return launch_mfma_nw<T, OutT, D, true, 8>(Q, K, V, O, ZH, S, scale_log2e, st);
    return launch_mfma_nw<T, OutT, D, true, 4>(Q, K, V, O, ZH, S, scale_log2e, st);
  }
  if (wide) return launch_mfma_nw<T, OutT, D, false, 8>(Q, K, V, O, ZH, S, scale_log2e, st);
  return launch_mfma_nw<T, OutT, D, false, 4>(Q, K, V, O, ZH, S, scale_log2e, st);
}

// head_dim < D: the 128-row form on padded tiles (the mask comes straight from global memory)
template <typename T, typename OutT, int D>
int launch_mfma_general(const void* Q, const void* K, const void* V, const void* mask, void* O, int64_t ZH, int64_t S,
                        int64_t Skv, float scale_log2e, hipStream_t st, int head_dim = D) {
  const float mask_factor = 1.44269504088896340736f / scale_log2e;     // mask / sm_scale
  if (head_dim < D) {
    const int64_t units = (S + 127) / 128 * ZH;
    if (units > 0x7fffffff) return HEXMI_ENOTSUP;
    const int64_t blocks = resident_grid(units, 2);
    if (blocks <= 0) return HEXMI_ELAUNCH;
    hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, D, false, true, 4, false, true>), dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                       static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(mask), (int)Skv,
                       mask_factor, 0, head_dim);
    return launch_status();
  }
  // a mask whose rows are whole 16-byte chunks is staged through LDS by 256-row workgroups (one per CU); the
  // copies address a workgroup's 256 mask rows with 32-bit byte offsets
  if (mask != nullptr && Skv % 8 == 0 && aligned_to(mask, 16) && S > 128 && Skv <= (1 << 21)) {
    const int64_t units8 = (S + 255) / 256 * ZH;
    if (units8 > 0x7fffffff) return HEXMI_ENOTSUP;
    const int64_t blocks8 = resident_grid(units8, 1);
    if (blocks8 <= 0) return HEXMI_ELAUNCH;
    hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, D, false, true, 8, true>), dim3((unsigned)blocks8), dim3(512), 0,
                       st, static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                       static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(mask), (int)Skv,
                       mask_factor);
    return launch_status();
  }
  const int64_t nqb = (S + 127) / 128;
  const int64_t units = nqb * ZH;
  if (units > 0x7fffffff) return HEXMI_ENOTSUP;
  const int64_t blocks = resident_grid(units, 2);
  if (blocks <= 0) return HEXMI_ELAUNCH;
  hipLaunchKernelGGL((flash_fwd_kernel<T, OutT, D, false, true>), dim3((unsigned)blocks), dim3(256), 0, st,
                     static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                     static_cast<OutT*>(O), (int)ZH, (int)S, scale_log2e, static_cast<const T*>(mask), (int)Skv,
                     mask_factor);
  return launch_status();
}

template <typename T, typename OutT>
int launch_rowwise(const void* Q, const void* K, const void* V, const void* mask, void* O, int64_t ZH, int64_t S,
                   int64_t Skv, int64_t D, float scale_log2e, bool causal, hipStream_t st) {
  const int64_t rows = ZH * S;
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffff || D > 256) return HEXMI_ENOTSUP;
  if (D <= 128)
    hipLaunchKernelGGL((flash_fwd_rowwise<T, OutT, 128>), dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                       static_cast<OutT*>(O), rows, (int)S, (int)D, scale_log2e, causal ? 1 : 0,
                       static_cast<const T*>(mask), (int)Skv);
  else                                                    // 256 output registers per lane: one wave per SIMD
    hipLaunchKernelGGL((flash_fwd_rowwise<T, OutT, 256>), dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const T*>(Q), static_cast<const T*>(K), static_cast<const T*>(V),
                       static_cast<OutT*>(O), rows, (int)S, (int)D, scale_log2e, causal ? 1 : 0,
                       static_cast<const T*>(mask), (int)Skv);
  return launch_status();
}

// mask == nullptr and Skv == S: the tuned kernels; otherwise the general ones.
template <typename T, typename OutT>
int dispatch_half(const void* Q, const void* K, const void* V, const void* mask, void* O, int64_t ZH, int64_t S,
                  int64_t Skv, int64_t D, float scale_log2e, bool causal, hipStream_t st) {
  // the matrix-core kernels address a head's keys with 32-bit byte offsets
  // and take the row maximum of the raw scores before scaling them, which is the maximum of the scaled scores only
  // for a positive scale: zero and negative scales go to the row-wise kernel, which scales first
  const bool ok = aligned_to(Q, 16) && aligned_to(K, 16) && aligned_to(V, 16) && aligned_to(O, 16) &&
                  Skv * D * (int64_t)sizeof(T) < 0x7fffffff && scale_log2e > 0.0f;
  const bool plain = !mask && Skv == S;
  if (ok && plain && D == 128) return launch_mfma<T, OutT, 128>(Q, K, V, O, ZH, S, scale_log2e, causal, st);
  if (ok && plain && D == 64) return launch_mfma<T, OutT, 64>(Q, K, V, O, ZH, S, scale_log2e, causal, st);
  // other head sizes up to 128 in multiples of 8 (rows on 16-byte boundaries): the same kernels on tiles padded with
  // zero columns to 64 or 128 ([2,16,2048,80] causal: 9.9 ms on the row-wise kernel)
  if (ok && plain && D % 8 == 0 && D < 128) {
    if (D < 64) {
      if (causal) return launch_mfma_padded<T, OutT, 64, true>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
      return launch_mfma_padded<T, OutT, 64, false>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
    }
    if (causal) return launch_mfma_padded<T, OutT, 128, true>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
    return launch_mfma_padded<T, OutT, 128, false>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
  }
  // ... and up to 256 as two halves of 128
  if (ok && plain && D % 8 == 0 && D > 128 && D <= 256) {
    if (causal) return launch_mfma_wide<T, OutT, true>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
    return launch_mfma_wide<T, OutT, false>(Q, K, V, O, ZH, S, (int)D, scale_log2e, st);
  }
  // (a mask is read in runs of four keys; without one any key count goes: cross-attention over 77 keys, say)
  const bool general_ok = ok && !causal && (!mask || (Skv % 4 == 0 && Skv >= 4 && aligned_to(mask, 8)));
  if (general_ok && D == 128) return launch_mfma_general<T, OutT, 128>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, st);
  if (general_ok && D == 64) return launch_mfma_general<T, OutT, 64>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, st);
  if (general_ok && D % 8 == 0 && D < 64) return launch_mfma_general<T, OutT, 64>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, st, (int)D);
  if (general_ok && D % 8 == 0 && D < 128) return launch_mfma_general<T, OutT, 128>(Q, K, V, mask, O, ZH, S, Skv, scale_log2e, st, (int)D);
  return launch_rowwise<T, OutT>(Q, K, V, mask, O, ZH, S, Skv, D, scale_log2e, causal, st);
}

int attention_any(const void* Q, const void* K, const void* V, const void* mask, void* O, int64_t ZH, int64_t S,
                  int64_t Skv, int64_t D, float sm_scale, bool cz, int in_dtype, int out_dtype, hipStream_t st) {
  const float c = sm_scale * 1.44269504088896340736f;
  if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F16) return dispatch_half<f16, f16>(Q, K, V, mask, O, ZH, S, Skv, D, c, cz, st);
  if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F32) return dispatch_half<f16, float>(Q, K, V, mask, O, ZH, S, Skv, D, c, cz, st);
  if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_BF16) return dispatch_half<bf16, bf16>(Q, K, V, mask, O, ZH, S, Skv, D, c, cz, st);
  if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_F32) return dispatch_half<bf16, float>(Q, K, V, mask, O, ZH, S, Skv, D, c, cz, st);
  if (in_dtype == HEXMI_F32 && out_dtype == HEXMI_F32) {
    int status = HEXMI_OK;
    if (flash_attn_f32_mfma(static_cast<const float*>(Q), static_cast<const float*>(K), static_cast<const float*>(V),
                            static_cast<const float*>(mask), static_cast<float*>(O), ZH, S, Skv, D, c, cz, st, &status))
      return status;
    return launch_rowwise<float, float>(Q, K, V, mask, O, ZH, S, Skv, D, c, cz, st);
  }
  return HEXMI_ENOTSUP;
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" int hexmi_flash_attn_fwd(const void* Q, const void* K, const void* V, void* O, int64_t Z, int64_t H,
                                    int64_t S, int64_t D, float sm_scale, int causal, int in_dtype, int out_dtype,
                                    hexmi_stream_t stream) {
  if (Z < 0 || H < 0 || S < 0 || D < 0) return HEXMI_EINVAL;
  if (Z == 0 || H == 0 || S == 0 || D == 0) return HEXMI_OK;
  if (!Q || !K || !V || !O) return HEXMI_EINVAL;
  if (S > 0x7fffffff / 2 || Z * H > 0x7fffffff) return HEXMI_ENOTSUP;
  begin_call();
  return attention_any(Q, K, V, nullptr, O, Z * H, S, S, D, sm_scale, causal != 0, in_dtype, out_dtype,
                       as_stream(stream));
}

extern "C" int hexmi_attention(const void* Q, const void* K, const void* V, const void* mask, void* O, int64_t batch,
                               int64_t seq_q, int64_t seq_kv, int64_t head_dim, float sm_scale, int in_dtype,
                               int out_dtype, hexmi_stream_t stream) {
  if (batch < 0 || seq_q < 0 || seq_kv < 0 || head_dim < 0) return HEXMI_EINVAL;
  if (batch == 0 || seq_q == 0 || head_dim == 0) return HEXMI_OK;
  if (seq_kv == 0) return HEXMI_EINVAL;                    // a softmax over no keys is undefined
  if (!Q || !K || !V || !O) return HEXMI_EINVAL;
  if (seq_q > 0x7fffffff / 2 || seq_kv > 0x7fffffff / 2 || batch > 0x7fffffff) return HEXMI_ENOTSUP;
  begin_call();
  return attention_any(Q, K, V, mask, O, batch, seq_q, seq_kv, head_dim, sm_scale, false, in_dtype, out_dtype,
                       as_stream(stream));
}
