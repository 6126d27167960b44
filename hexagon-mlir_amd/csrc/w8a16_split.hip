// W8A16 for up to 256 activation rows on a two-dimensional decomposition: a workgroup owns a range of output
// channels AND a range of K, so that (row tiles x channel ranges x K parts) comes to about the number of compute units
// whatever N is (N = 4096, K = 11008 on 256 CUs: 64 ranges of 64 channels x 4 K parts at M <= 128). Against one
// channel range per CU over all of K this divides the activation traffic through L2 by the number of K parts (a
// workgroup reads only its K part of A), and it keeps every CU busy when N / 48 or (M / 128) x (N / 128) is far from
// the CU count, which is what the kernels of w8a16.hip and the tiled GEMM need.
//
// Workgroup = 8 waves = 4 channel groups x 2 K halves of every 128-k slab. A wave owns CT tiles of 16 channels for
// all RB blocks of 16 activation rows: it loads its weights global -> registers (16 bytes per lane: 16 rows x 64
// bytes per instruction, three slabs ahead), widens them to fp16 once per slab (exact), one slab ahead and spread
// between the matrix instructions, and multiplies them against every row block: 16 * CT conversions for
// 2 * RB * CT matrix instructions. Activations go global -> LDS (global_load_lds, three stages, one barrier per slab)
// and every wave reads the fragments of its K half.
//
// The K parts of a tile are summed through a caller workspace. Parts 0 .. P-2 write their fp32 partial tiles with
// write-through stores, wait until those are counted off and raise a flag each; part P-1, whose workgroups have the
// highest indices and so are dispatched last, waits for the flags (a bounded wait: the parts it waits for never
// wait for anything), adds the partial tiles in the order 0, 1, ... with its own last, applies the channel scales and
// stores fp16. The order does not depend on the channel, on the workgroup or on timing: results are reproducible bit
// for bit and permuting channels permutes columns. XCDs have separate L2 caches: a flag carries its writer's XCD,
// and the reader takes a partial tile from its own L2 when that is the same XCD and past the caches otherwise.
#include <type_traits>
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr int kSlab = 128;                                  // k per slab: 64 per K half
constexpr int kCG = 4, kKH = 2;                             // channel groups x K halves = 8 waves
constexpr int kThreads = kCG * kKH * kWave;
constexpr int kMaxCT = 3;
constexpr unsigned kSpinLimit = 1u << 22;                   // polls of a counter before a workgroup gives up
// bytes of one partial tile in the workspace: eight wave regions of (row blocks / 2, at least one) x ct KiB; the
// kernel's indexing and the size the host asks the caller for both come from here
constexpr int split_tile_bytes(int rb, int ct) { return kCG * kKH * (rb >= 2 ? rb / 2 : 1) * ct * 1024; }

#define HEXMI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define HEXMI_GLB(p) ((const __attribute__((address_space(1))) void*)(p))
#define HEXMI_FENCE __builtin_amdgcn_sched_barrier(0)

// s_waitcnt immediate (gfx9 encoding): at most vm vector-memory operations outstanding, other counters untouched
constexpr int wait_vm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

struct SplitArgs {
  const f16* A;
  const int8_t* W;
  const f16* scales;
  f16* C;
  int M, N, K;
  int chan_per_wg, col_tiles, row_tiles, parts;
  float* partials;                                          // [part][tile][wave][HB][CT][64 lanes][4]
  unsigned partial_bytes;                                   // size of that area: the buffer descriptor's bound
  unsigned* counters;                                       // [tiles][parts]: nonzero once a part's partial tile is out
  unsigned* error;                                          // word 0 of the workspace: set when a bounded wait ran out
};

template <int RB, int CT>
__global__ __launch_bounds__(kThreads)
void w8a16_split_kernel(const SplitArgs p) {
  constexpr int ROWS = RB * 16;
  constexpr int STAGE = ROWS * kSlab;                       // fp16 elements of one activation stage
  constexpr int NA = RB * 4;                                // 1 KiB copies per slab (4 rows of 256 bytes each)
  constexpr int NAW = NA >= 8 ? NA / 8 : 1;                 // per wave; with fewer than 8 copies some are issued twice
  __shared__ __attribute__((aligned(16))) f16 a_s0[STAGE];
  __shared__ __attribute__((aligned(16))) f16 a_s1[STAGE];
  __shared__ __attribute__((aligned(16))) f16 a_s2[STAGE];
  __shared__ __attribute__((aligned(16))) float red3[RB * CT * 256];   // K-half partial of channel group 3
  __shared__ unsigned same_s;
  static_assert(RB * CT * 1024 <= STAGE * 2, "a wave's partial tile fits one activation stage");

  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int r16 = lane % 16, kg = lane / 16;
  const int cg = wave % kCG, kh = wave / kCG;

  const int ctile = blockIdx.x % p.col_tiles;
  const int rtile = (blockIdx.x / p.col_tiles) % p.row_tiles;
  const int part = blockIdx.x / (p.col_tiles * p.row_tiles);
  const int K = p.K;
  const int n_begin = ctile * p.chan_per_wg;
  const int n_end = n_begin + p.chan_per_wg < p.N ? n_begin + p.chan_per_wg : p.N;
  const int m0 = rtile * ROWS;
  // K parts in whole slabs, the first (slabs % parts) of them one slab longer: the same split for every tile
  const int total_slabs = K / kSlab;
  const int q = total_slabs / p.parts, rem = total_slabs % p.parts;
  const int slab0 = part * q + (part < rem ? part : rem);
  const int n_slabs = q + (part < rem ? 1 : 0);

  // channel tiles of this wave that hold at least one channel (wave-uniform)
  int nct = 0;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
    if (n_begin + (cg * CT + ct) * 16 < n_end) nct = ct + 1;

  // the channel scales of this lane's outputs, requested first: they come from HBM
  f16 sc[CT][4];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int gn = n_begin + (cg * CT + ct) * 16 + kg * 4 + e;
      sc[ct][e] = p.scales[gn < n_end ? gn : n_end - 1];
    }

  // ---- weights: lane (r16, kg) of tile ct reads bytes [64 kh + 16 kg, +16) of every slab of its channel's row
  const int8_t* wp[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    int n = n_begin + (cg * CT + ct) * 16 + r16;
    n = n < n_end ? n : n_end - 1;                          // past the range: its last row again, results dropped
    wp[ct] = p.W + (int64_t)n * K + (int64_t)slab0 * kSlab + kh * 64 + kg * 16;
  }
  auto slab_at = [&](int j) { return j < n_slabs ? j : n_slabs - 1; };   // past the end: the last slab again, unused
  // where the loads past the end of the K part go: kMaxCT KiB of the activation matrix, a different place for
  // every wave of the grid so that they do not all queue on the same L2 lines
  const char* idle_src;
  {
    const int64_t a_bytes = (int64_t)p.M * K * 2;
    const int64_t spots = a_bytes >= (kMaxCT + 1) * 1024 ? (a_bytes - kMaxCT * 1024) / 1024 : 1;
    idle_src = reinterpret_cast<const char*>(p.A) + (((int64_t)blockIdx.x * (kCG * kKH) + wave) % spots) * 1024 + lane * 16;
  }

  // ---- activations: a copy moves 4 rows x 256 bytes; the 16-byte chunk c of row r sits at position c ^ (r % 16)
  const f16* a_src[NAW];
  int a_dst[NAW];
#pragma unroll
  for (int i = 0; i < NAW; ++i) {
    const int inst = (i * 8 + wave) % NA;
    const int row = inst * 4 + lane / 16;
    const int chunk = (lane % 16) ^ (row & 15);
    const int gm = m0 + row < p.M ? m0 + row : p.M - 1;
    a_src[i] = p.A + (int64_t)gm * K + (int64_t)slab0 * kSlab + chunk * 8;
    a_dst[i] = inst * 512;
  }
  auto copy_a = [&](int j, f16* stage) __attribute__((always_inline)) {
    const int64_t off = (int64_t)slab_at(j) * kSlab;
#pragma unroll
    for (int i = 0; i < NAW; ++i)
      __builtin_amdgcn_global_load_lds(HEXMI_GLB(a_src[i] + off), HEXMI_LDS(stage + a_dst[i]), 16, 0, 0);
  };
  // fragment of row block rb, step t (32 k): row rb*16 + r16, chunk 8 kh + 2 kg + t
  const int a_off0 = (r16 * 16 + ((8 * kh + 2 * kg) ^ r16)) * 8;
  const int a_off1 = (r16 * 16 + ((8 * kh + 2 * kg + 1) ^ r16)) * 8;

  f32x4 acc[RB][CT];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[rb][ct] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The K loop, written once per number NCT of channel tiles the wave really has (the last group of a range may hold
  // fewer than CT): straight-line code without a branch per tile.
  // The weights of slab j+1 are widened to fp16 during slab j, a few instructions after each row block's MFMAs
  // (vector and matrix instructions overlap; a conversion phase at the head of the slab would leave the matrix pipe
  // idle in every wave at once, since the barrier lines the waves up): raw weights sit in three register slots
  // (slab j in slot j % 3, refilled with slab j+3 once converted), fp16 fragments in two.
  // Issue order, which the wait counts rely on: W(0) W(1) A(0) W(2) A(1) W(3), then slab j: A(j+2) ... W(j+4).
  // A(j) is followed by W(j+2), A(j+1), W(j+3): 2 NCT + NAW younger operations when slab j starts; W(j+1), which
  // slab j converts, is older than A(j).
  auto k_loop = [&](auto nct_tag) __attribute__((always_inline)) {
    constexpr int NCT = decltype(nct_tag)::value;
    constexpr int NC1 = NCT > 0 ? NCT : 1;
    u32x4 raw[3][NC1];
    u32x4 bf[2][NC1][2];                                    // fp16 fragments as dwords: [buffer][tile][step]
    auto load_w = [&](int j, u32x4* dst) __attribute__((always_inline)) {
      const int64_t off = (int64_t)slab_at(j) * kSlab;
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct)
        dst[ct] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp[ct] + off));
    };
    // the same number of loads from a place that is certain to hit L2, results never used
    auto load_idle = [&](u32x4* dst) __attribute__((always_inline)) {
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct)
        dst[ct] = *reinterpret_cast<const u32x4*>(idle_src + ct * 1024);
    };
    // dwords [d0, d1) of a slab's 4 * NCT raw dwords -> fragments
    auto widen = [&](const u32x4* w, u32x4 (*dst)[2], int d0, int d1) __attribute__((always_inline)) {
#pragma unroll
      for (int d = 0; d < 4 * NCT; ++d)
        if (d >= d0 && d < d1) {
          uint32_t lo, hi;
          cvt4(w[d / 4][d % 4], lo, hi);
          dst[d / 4][(d % 4) / 2][(d % 2) * 2] = lo;
          dst[d / 4][(d % 4) / 2][(d % 2) * 2 + 1] = hi;
        }
    };
    HEXMI_FENCE;
    load_w(0, raw[0]);
    load_w(1, raw[1]);
    HEXMI_FENCE;
    copy_a(0, a_s0);
    HEXMI_FENCE;
    load_w(2, raw[2]);
    HEXMI_FENCE;
    copy_a(1, a_s1);
    HEXMI_FENCE;
    widen(raw[0], bf[0], 0, 4 * NCT);
    HEXMI_FENCE;
    load_w(3, raw[0]);
    HEXMI_FENCE;
    // last_slabs: one of the last slabs of this K part, whose loads may lie past its end. Every slab issues the
    // same copies and loads (the waits count them); past the end the activation copy repeats the last slab, an L2
    // hit, and the weight load reads a piece of the activation matrix instead, which every workgroup has just
    // pulled through L2: re-reading the last weight slab would be another trip to HBM (they are read past the
    // caches), four slabs out of a K part's dozen or two, and the end of the loop would wait for it.
    auto slab = [&](int j, const f16* cur, f16* fill, u32x4 (*bcur)[2], u32x4 (*bnxt)[2], u32x4* wnxt,
                    auto last_slabs) __attribute__((always_inline)) {
      constexpr bool LAST = decltype(last_slabs)::value;
      HEXMI_FENCE;
      __builtin_amdgcn_s_waitcnt(wait_vm(2 * NCT + NAW));   // own copies of slab j have landed (and W(j+1))
      __builtin_amdgcn_s_barrier();                         // everyone's have; the stage of slab j-1 is free
      HEXMI_FENCE;
      copy_a(j + 2, fill);
      HEXMI_FENCE;
      if constexpr (NCT > 0) {
        // Row blocks in groups of GR: the fragments of group g+1 are requested before the arithmetic of group g and
        // waited for with a count that leaves them in flight (left to the compiler, every row block waited for the
        // reads it had just issued: a full LDS latency eight times per slab), and a group's MFMAs run step 0 of
        // all its row blocks, then step 1, so that independent MFMAs lie between two that update the
        // same accumulator (GR * NCT >= 3: a 16x16x32 MFMA is in the pipe for two issue slots of 16 cycles). The reads are
        // assembly for the reason given at wait_group.
        constexpr int GW = NCT >= 3 ? 1 : NCT == 2 ? 2 : 4;   // three or four MFMAs between two on one accumulator
        constexpr int GR = RB < GW ? RB : GW;
        constexpr int NG = RB / GR;
        static_assert(RB % GR == 0, "whole groups");
        u32x4 fa[2][GR][2];                                 // [buffer][row block of the group][step]
        const unsigned at0 = (unsigned)(size_t)(__attribute__((address_space(3))) const char*)(cur) + a_off0 * 2;
        const unsigned at1 = (unsigned)(size_t)(__attribute__((address_space(3))) const char*)(cur) + a_off1 * 2;
        auto read_group = [&](int g, u32x4 (*dst)[2]) __attribute__((always_inline)) {
#pragma unroll
          for (int i = 0; i < GR; ++i) {
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst[i][0]) : "v"(at0), "n"((g * GR + i) * 16 * kSlab * 2) : "memory");
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(dst[i][1]) : "v"(at1), "n"((g * GR + i) * 16 * kSlab * 2) : "memory");
          }
        };
        // waits until at most `newer` LDS reads are outstanding; names the group's registers as modified so that
        // nothing that uses them is scheduled above the wait (and nothing moves them while their reads are in flight)
        auto wait_group = [&](u32x4 (*f)[2], auto newer) __attribute__((always_inline)) {
          constexpr int NEWER = decltype(newer)::value;
          if constexpr (GR == 1)
            asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(f[0][0]), "+v"(f[0][1]) : "n"(NEWER) : "memory");
          else if constexpr (GR == 2)
            asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[1][0]), "+v"(f[1][1]) : "n"(NEWER) : "memory");
          else
            asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[1][0]), "+v"(f[1][1]), "+v"(f[2][0]),
                         "+v"(f[2][1]), "+v"(f[3][0]), "+v"(f[3][1]) : "n"(NEWER) : "memory");
        };
        read_group(0, fa[0]);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          u32x4 (*fc)[2] = fa[g % 2];
          if (g + 1 < NG) {
            read_group(g + 1, fa[(g + 1) % 2]);
            wait_group(fc, std::integral_constant<int, 2 * GR>{});
          } else {
            wait_group(fc, std::integral_constant<int, 0>{});
          }
          // D[i = channel][j = activation row]: lane holds row j = lane%16, channels 4*(lane/16) + 0..3
#pragma unroll
          for (int st = 0; st < 2; ++st)
#pragma unroll
            for (int i = 0; i < GR; ++i)
#pragma unroll
              for (int ct = 0; ct < NCT; ++ct)
                acc[g * GR + i][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    __builtin_bit_cast(f16x8, bcur[ct][st]), __builtin_bit_cast(f16x8, fc[i][st]), acc[g * GR + i][ct], 0, 0, 0);
          widen(wnxt, bnxt, g * GR * 4 * NCT / RB, (g + 1) * GR * 4 * NCT / RB);
          HEXMI_FENCE;
        }
      }
      HEXMI_FENCE;
      if (LAST && j + 4 >= n_slabs) load_idle(wnxt);
      else load_w(j + 4, wnxt);
      HEXMI_FENCE;
    };
    // Whole rounds of six slabs (three stages and raw slots, two fragment buffers) as long as every slab of the
    // round still has four behind it, then the up to nine that are left, each with the tests of a last slab: no
    // exit from the middle of a round (with one, the compiler loses count of the loads in flight at the loop head
    // and waits for all of them).
    constexpr std::false_type kBody{};
    constexpr std::true_type kLast{};
    int j = 0;
    for (; j + 10 <= n_slabs; j += 6) {
      slab(j, a_s0, a_s2, bf[0], bf[1], raw[1], kBody);
      slab(j + 1, a_s1, a_s0, bf[1], bf[0], raw[2], kBody);
      slab(j + 2, a_s2, a_s1, bf[0], bf[1], raw[0], kBody);
      slab(j + 3, a_s0, a_s2, bf[1], bf[0], raw[1], kBody);
      slab(j + 4, a_s1, a_s0, bf[0], bf[1], raw[2], kBody);
      slab(j + 5, a_s2, a_s1, bf[1], bf[0], raw[0], kBody);
    }
    if (j < n_slabs) slab(j, a_s0, a_s2, bf[0], bf[1], raw[1], kLast);
    if (j + 1 < n_slabs) slab(j + 1, a_s1, a_s0, bf[1], bf[0], raw[2], kLast);
    if (j + 2 < n_slabs) slab(j + 2, a_s2, a_s1, bf[0], bf[1], raw[0], kLast);
    if (j + 3 < n_slabs) slab(j + 3, a_s0, a_s2, bf[1], bf[0], raw[1], kLast);
    if (j + 4 < n_slabs) slab(j + 4, a_s1, a_s0, bf[0], bf[1], raw[2], kLast);
    if (j + 5 < n_slabs) slab(j + 5, a_s2, a_s1, bf[1], bf[0], raw[0], kLast);
    if (j + 6 < n_slabs) slab(j + 6, a_s0, a_s2, bf[0], bf[1], raw[1], kLast);
    if (j + 7 < n_slabs) slab(j + 7, a_s1, a_s0, bf[1], bf[0], raw[2], kLast);
    if (j + 8 < n_slabs) slab(j + 8, a_s2, a_s1, bf[0], bf[1], raw[0], kLast);
  };
  if (nct == CT) k_loop(std::integral_constant<int, CT>{});
  else if (CT > 2 && nct == 2) k_loop(std::integral_constant<int, (CT > 2 ? 2 : 0)>{});
  else if (CT > 1 && nct == 1) k_loop(std::integral_constant<int, (CT > 1 ? 1 : 0)>{});
  else k_loop(std::integral_constant<int, 0>{});
  HEXMI_FENCE;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");           // trailing copies land before the stages are reused
  __syncthreads();

  // ---- the two K halves of a tile exchange halves of their row blocks through LDS: afterwards wave (cg, kh) holds the
  //      finished sums of row blocks [kh * HB, (kh + 1) * HB) and all eight waves share the rest of the work.
  //      (A single row block stays with half 0.)
  constexpr int HB = RB >= 2 ? RB / 2 : 1;
  constexpr int kRegion = HB * CT * 256;                    // floats a wave hands over
  const bool active = RB >= 2 || kh == 0;
  const int rb0 = RB >= 2 ? kh * HB : 0;
  // LDS region wave w receives in: two per activation stage and the last two in red3 (a single row block: one per
  // stage, the fourth in red3; only half 0 receives)
  auto region = [&](int w) {
    if constexpr (RB == 1) {
      return w == 0 ? reinterpret_cast<float*>(a_s0) : w == 1 ? reinterpret_cast<float*>(a_s1)
             : w == 2 ? reinterpret_cast<float*>(a_s2) : red3;
    } else {
      float* base = w < 2 ? reinterpret_cast<float*>(a_s0) : w < 4 ? reinterpret_cast<float*>(a_s1)
                    : w < 6 ? reinterpret_cast<float*>(a_s2) : red3;
      return base + (w % 2) * kRegion;
    }
  };
  {
    static_assert(RB == 1 ? kRegion * 4 <= STAGE * 2 : 2 * kRegion * 4 <= STAGE * 2 && 2 * kRegion <= RB * CT * 256, "regions fit");
    const int partner = cg + (1 - kh) * kCG;
    if (RB >= 2 || kh == 1) {                                // hand over the row blocks the partner finishes
      float* dst = region(partner);
      const int give0 = RB >= 2 ? (1 - kh) * HB : 0;
#pragma unroll
      for (int h = 0; h < HB; ++h)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          f32x4 v = acc[0][ct];
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            if (rb == give0 + h) v = acc[rb][ct];
          *reinterpret_cast<f32x4*>(dst + ((h * CT + ct) * 64 + lane) * 4) = v;
        }
    }
    __syncthreads();
  }
  f32x4 fin[HB][CT];                                        // this wave's finished (or, with K parts, partial) sums
  {
    const float* src = region(wave < 8 ? wave : 0);
#pragma unroll
    for (int h = 0; h < HB; ++h)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        f32x4 own = acc[0][ct];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          if (rb == rb0 + h) own = acc[rb][ct];
        // K half 0 first, then half 1: the same order in both waves
        const f32x4 other = active ? *reinterpret_cast<const f32x4*>(src + ((h * CT + ct) * 64 + lane) * 4) : own;
        fin[h][ct] = kh == 0 ? own + other : other + own;
      }
  }
  // ---- the K parts of a tile, through the workspace. Part parts-1 adds them up, in the order 0, 1, ... with its own
  //      last; its workgroups have the highest indices, so the parts it waits for were dispatched before it.
  if (p.parts > 1) {
    const int tiles = p.col_tiles * p.row_tiles;
    const int tile = rtile * p.col_tiles + ctile;
    unsigned* flags = p.counters + tile * p.parts;
    constexpr int kTileBytes = split_tile_bytes(RB, CT);    // eight wave regions (a single row block uses four of them)
    static_assert(kTileBytes == kCG * kKH * kRegion * 4, "the regions fill a partial tile");
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(xcc));
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>(p.partials), 0, (int)p.partial_bytes, 0x00020000);
    // (bounded by the area's size: an access past it is dropped by the hardware instead of landing in someone's memory)
    const int wave_off = (RB >= 2 ? wave : cg) * kRegion * 4 + lane * 16;
    constexpr int kThrough = 1 | (1 << 4);                  // sc0 sc1: system scope, past both cache levels
    constexpr int kDevice = 1 << 4;                         // sc1: device scope, served by this XCD's L2
    if (part + 1 < p.parts) {
      // Writer: the partial tile goes out with write-through stores; when they have been counted off the data is
      // where every XCD sees it (a workgroup barrier alone does not wait for stores), and the flag says so.
      if (active) {
        const int base = (part * tiles + tile) * kTileBytes + wave_off;
#pragma unroll
        for (int h = 0; h < HB; ++h)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, fin[h][ct]), rsrc,
                                                       base + (h * CT + ct) * 1024, 0, kThrough);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (threadIdx.x == 0) __hip_atomic_store(flags + part, 0x100u | xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      return;
    }
    // Reducer. A writer on this XCD left its lines in the L2 this workgroup reads through; lines written on another
    // XCD are fetched past the caches.
    if (threadIdx.x == 0) {
      unsigned same = 0;
      for (int sp = 0; sp + 1 < p.parts; ++sp) {
        unsigned f = 0, polls = 0;
        while ((f = __hip_atomic_load(flags + sp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)) == 0) {
          __builtin_amdgcn_s_sleep(1);
          if (++polls > kSpinLimit) {                        // never seen; every wave still leaves the kernel
            __hip_atomic_store(p.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
          }
        }
        if (f == (0x100u | xcc)) same |= 1u << sp;
        // back to zero: the workspace is ready for the next call
        __hip_atomic_store(flags + sp, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
      same_s = same;
    }
    __syncthreads();
    if (active) {
      const unsigned same = same_s;
      f32x4 sum[HB][CT];
      for (int sp = 0; sp + 1 < p.parts; ++sp) {
        const int base = (sp * tiles + tile) * kTileBytes + wave_off;
        const bool local = (same >> sp) & 1u;
#pragma unroll
        for (int h = 0; h < HB; ++h)
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) {
            const u32x4 v = local ? __builtin_amdgcn_raw_buffer_load_b128(rsrc, base + (h * CT + ct) * 1024, 0, kDevice)
                                  : __builtin_amdgcn_raw_buffer_load_b128(rsrc, base + (h * CT + ct) * 1024, 0, kThrough);
            const f32x4 f = __builtin_bit_cast(f32x4, v);
            sum[h][ct] = sp == 0 ? f : sum[h][ct] + f;
          }
      }
#pragma unroll
      for (int h = 0; h < HB; ++h)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) fin[h][ct] = sum[h][ct] + fin[h][ct];
    }
  }
  if (active) {
#pragma unroll
    for (int h = 0; h < HB; ++h) {
      const int gm = m0 + (rb0 + h) * 16 + r16;
      if (gm >= p.M) continue;
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const int gn = n_begin + (cg * CT + ct) * 16 + kg * 4;
        f16* dst = p.C + (int64_t)gm * p.N + gn;
        if (gn + 4 <= n_end) {
          store4<f16>(dst, fin[h][ct][0] * (float)sc[ct][0], fin[h][ct][1] * (float)sc[ct][1],
                      fin[h][ct][2] * (float)sc[ct][2], fin[h][ct][3] * (float)sc[ct][3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (gn + e < n_end) dst[e] = (f16)(fin[h][ct][e] * (float)sc[ct][e]);
        }
      }
    }
  }
}
#undef HEXMI_LDS
#undef HEXMI_GLB
#undef HEXMI_FENCE

__global__ void zero_words_kernel(unsigned* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// The decomposition for (M, N, K) on `cus` compute units; parts == 0: this kernel does not take the shape.
struct SplitPlan {
  int rb, ct, row_tiles, col_tiles, chan_per_wg, parts;
  int64_t header_bytes, bytes;
};

inline int round_up(int64_t v, int to) { return (int)((v + to - 1) / to * to); }

SplitPlan plan_split(int64_t M, int64_t N, int64_t K, int cus) {
  SplitPlan pl = {};
  if (M < 1 || M > 256 || N < 16 || N % 4 != 0 || K < kSlab || K % kSlab != 0 || cus <= 0) return pl;
  if (N > (1 << 24) || K > (1 << 24)) return pl;
  if (M * K * 2 < (kMaxCT + 1) * 1024) return pl;           // the kernel's idle loads read that much of A
  pl.rb = M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8;
  pl.row_tiles = (int)((M + pl.rb * 16 - 1) / (pl.rb * 16));
  const int slabs = (int)(K / kSlab);
  const int min_cols = (int)((N + kMaxCT * 64 - 1) / (kMaxCT * 64));
  // as many K parts as it takes for the grid to reach the CU count with the widest channel ranges (the narrower
  // the ranges, the more often A crosses L2); at most 8, each of three slabs or more
  int parts = 1;
  while (parts < 8 && pl.row_tiles * min_cols * parts * 2 <= cus && slabs / (parts * 2) >= 3) parts *= 2;
  if (parts > slabs) parts = slabs;
  int cols = cus / (pl.row_tiles * parts);
  if (cols < min_cols) cols = min_cols;
  int chan = round_up((N + cols - 1) / cols, 4);
  if (chan < 16) chan = 16;
  cols = (int)((N + chan - 1) / chan);
  pl.parts = parts;
  pl.col_tiles = cols;
  pl.chan_per_wg = chan;
  pl.ct = (chan + 63) / 64;
  const int64_t tiles = (int64_t)cols * pl.row_tiles;
  pl.header_bytes = round_up((tiles * parts + 1) * 4, 256);
  pl.bytes = parts > 1 ? pl.header_bytes + (int64_t)parts * tiles * split_tile_bytes(pl.rb, pl.ct) : 0;
  return pl;
}

template <int RB>
int launch_split_ct(const SplitPlan& pl, const SplitArgs& args, hipStream_t st) {
  const dim3 grid((unsigned)(pl.col_tiles * pl.row_tiles * pl.parts));
  if (pl.ct == 1) hipLaunchKernelGGL((w8a16_split_kernel<RB, 1>), grid, dim3(kThreads), 0, st, args);
  else if (pl.ct == 2) hipLaunchKernelGGL((w8a16_split_kernel<RB, 2>), grid, dim3(kThreads), 0, st, args);
  else hipLaunchKernelGGL((w8a16_split_kernel<RB, 3>), grid, dim3(kThreads), 0, st, args);
  return launch_status();
}

}  // namespace

int64_t w8a16_split_workspace(int64_t M, int64_t N, int64_t K, int cus) { return plan_split(M, N, K, cus).bytes; }
int64_t w8a16_split_header(int64_t M, int64_t N, int64_t K, int cus) { return plan_split(M, N, K, cus).header_bytes; }

// true: the split kernel took the call (status in *status)
bool w8a16_split(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales, f16* C,
                 void* workspace, int64_t workspace_bytes, int cus, hipStream_t st, int* status) {
  const SplitPlan pl = plan_split(M, N, K, cus);
  if (pl.parts == 0) return false;
  if (pl.parts > 1 && (!workspace || workspace_bytes < pl.bytes)) return false;
  if (!aligned_to(A, 16) || !aligned_to(W, 16) || !aligned_to(C, 8) || !aligned_to(workspace, 16)) return false;
  SplitArgs args;
  args.A = A; args.W = W; args.scales = scales; args.C = C;
  args.M = (int)M; args.N = (int)N; args.K = (int)K;
  args.chan_per_wg = pl.chan_per_wg; args.col_tiles = pl.col_tiles; args.row_tiles = pl.row_tiles; args.parts = pl.parts;
  args.error = static_cast<unsigned*>(workspace);          // word 0: where a caller can find it
  args.counters = args.error + 1;
  args.partials = reinterpret_cast<float*>(static_cast<char*>(workspace) + pl.header_bytes);
  args.partial_bytes = (unsigned)(pl.bytes > pl.header_bytes ? pl.bytes - pl.header_bytes : 0);
  if (pl.rb == 1) *status = launch_split_ct<1>(pl, args, st);
  else if (pl.rb == 2) *status = launch_split_ct<2>(pl, args, st);
  else if (pl.rb == 4) *status = launch_split_ct<4>(pl, args, st);
  else *status = launch_split_ct<8>(pl, args, st);
  return true;
}

int w8a16_split_clear(void* workspace, int64_t bytes, hipStream_t st) {
  const int n = (int)(bytes / 4);
  hipLaunchKernelGGL(zero_words_kernel, dim3((n + 255) / 256), dim3(256), 0, st, static_cast<unsigned*>(workspace), n);
  return launch_status();
}

}  // namespace hexmi
