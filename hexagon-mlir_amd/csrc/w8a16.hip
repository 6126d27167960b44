// Weight-only int8 GEMM (W8A16): C[m,n] = scale[n] * sum_k A[m,k] * W[n,k], fp16 activations, int8 weights,
// fp32 accumulation on 16x16x32 matrix-core tiles, fp16 output.
//
// The weight matrix is the only large operand (N*K bytes) and every weight is used once per 16 activation rows,
// so weights never touch LDS: each lane fetches 16 consecutive int8 of one output channel straight from HBM
// (16-byte loads, a 16-channel tile reads 64 contiguous bytes per channel per instruction), converts them to
// fp16 in registers (exact: one v_cvt_f16_i16 per weight on the sign-extended byte) and feeds two MFMAs.
//
// The per-channel scale multiplies the finished fp32 sum (it is constant over k), which differs from
// "dequantise, then multiply" only by fp32 rounding; hexmi_dequant_w8 exposes the element-wise dequantisation.
//
// Work split: a workgroup of 4 waves owns one tile of 16 output channels; the waves split K four ways and their
// partial tiles are summed through LDS.
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * kWave;

// One workgroup (4 waves) per tile of 16 output channels; wave w owns the K range [w*K/4, (w+1)*K/4) in steps of
// 64 (one 16-byte weight load per lane = two MFMAs). All weight loads of a round are issued before the first
// conversion so a wave keeps up to 8 KiB of the weight stream in flight; with every tile a separate workgroup
// the whole grid is resident at once and nothing synchronises across tiles. Activation fragments are read
// through L1/L2 (the activations are M*K*2 bytes, at most 128 KiB per 16 rows, shared by every workgroup).
// MT: number of 16-row activation tiles handled per pass (rows m_base .. m_base + 16*MT).
// ZP: the asymmetric forms of quant.dcast, f = (float(q) - zero_point) * scale with per-channel or per-tensor
// parameters: the zero point (an int8, exact in fp16, as is every difference q - zero_point) is subtracted from the
// widened weights; per_tensor reads scale and zero point at index 0 for every channel.
template <int MT, bool ZP = false>
__global__ __launch_bounds__(kThreads)
void w8a16_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                  f16* __restrict__ C, int M, int N, int K, int m_base, const int8_t* __restrict__ zero_points = nullptr,
                  int per_tensor = 0) {
  __shared__ __attribute__((aligned(16))) float red[kWaves * MT * 256];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r16 = lane % 16, kg = lane / 16;               // tile row / 16-byte k group of this lane
  const int tile = blockIdx.x;
  const int n = tile * 16 + r16;
  const int nc = n < N ? n : N - 1;
  const int8_t* wrow = W + (int64_t)nc * K + kg * 16;
  f16 zp_h = (f16)0.0f;
  if constexpr (ZP) {
    if (zero_points) zp_h = (f16)(float)zero_points[per_tensor ? 0 : nc];
  }

  const int steps = K / 64;
  const int per_wave = (steps + kWaves - 1) / kWaves;       // consecutive steps per wave: whole 128-byte lines
  const int s_begin = wave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;

  const f16* arow[MT];
  bool avalid[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int gm = m_base + t * 16 + r16;
    avalid[t] = gm < M;
    arow[t] = A + (int64_t)(avalid[t] ? gm : 0) * K + kg * 16;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // A round issues U weight loads and the 2*U*MT activation loads that go with them before anything is
  // consumed, so the HBM latency of the weights and the L2 latency of the activations overlap.
  constexpr int U = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
  for (int s0 = s_begin; s0 < s_end; s0 += U) {
    u32x4 wv[U];
    f16x8 av[U][MT][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      if (s0 + u < s_end) wv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + (int64_t)(s0 + u) * 64));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (s0 + u) * 64;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        av[u][t][0] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        av[u][t][1] = av[u][t][0];
        if (avalid[t] && s0 + u < s_end) {
          av[u][t][0] = *reinterpret_cast<const f16x8*>(arow[t] + k);
          av[u][t][1] = *reinterpret_cast<const f16x8*>(arow[t] + k + 8);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      f16x8 w0, w1;
      cvt16(wv[u], w0, w1);                                 // a skipped step has zero weights and activations
      if constexpr (ZP) {
        w0 -= zp_h;                                         // exact: integers of magnitude <= 255
        w1 -= zp_h;
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        // D[i = channel][j = activation row]: lane holds row j = lane%16, channels 4*(lane/16) + 0..3
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, av[u][t][0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, av[u][t][1], acc[t], 0, 0, 0);
      }
    }
  }

  // sum the K-partials of the waves
#pragma unroll
  for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4*>(red + ((wave * MT + t) * 64 + lane) * 4) = acc[t];
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
        if (gn + e < N) C[(int64_t)gm * N + gn + e] = (f16)(sum[e] * (float)scales[ZP && per_tensor ? 0 : gn + e]);
    }
  }
}

// Up to 16 activation rows on pre-packed weights, K <= 4096 (plain weights go through the chunked kernel further
// down, which is faster at every row count: 11.3 against 11.8-12.3 us at M = 4 and 8, N = 11008, K = 4096; 6.9
// against 8.6 at N = K = 4096): persistent workgroups of 16 waves, one per compute unit. The per-CU rate
// of the weight reads is what bounds this shape, so the output channels are dealt in equal
// contiguous ranges over exactly as many workgroups as there are CUs (N = 11008 on 256 CUs: 43 channels each,
// walked as tiles of 16, 16 and 11 channels; the lanes of a short tile re-read its last row and drop the result).
// Wave w owns the K slice [w*K/16, (w+1)*K/16) of every tile of its workgroup: it needs only a 16 x K/16 slice of
// the activations, which it keeps in registers for all its tiles (no LDS staging, activations cross L2 once per
// workgroup), and it issues the weight loads of all its tiles up front so the whole weight matrix is requested at
// kernel start. The 16 K-partials of a tile are summed through LDS.
// Measured alternatives that were no faster: fully contiguous 1 KiB row copies into LDS (global_load_lds) with
// swizzled fragment reads (the better HBM pattern is paid back in barriers), and issuing the activation loads
// first. The activation slices themselves (128 KiB per CU from L2 at M = 16) cost about 2 us of the 14.
constexpr int kPWaves = 16;
constexpr int kPTiles = 3;                                  // tiles per workgroup per pass
constexpr int kPSteps = 4;                                  // 64-wide steps per wave: K <= 16 * 4 * 64
// W is the fragment-major layout written by pack_w8_kernel (chan_per_wg is a multiple of 16): the 16 rows x 64 k
// of a tile step are one contiguous KiB in lane order, so a wave's loads are fully contiguous.
__global__ __launch_bounds__(1024)
void w8a16_persist_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                          f16* __restrict__ C, int M, int N, int K, int chan_per_wg) {
  __shared__ __attribute__((aligned(16))) float red[kPTiles * kPWaves * 256];   // [slot][wave][lane][4]

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r16 = lane % 16, kg = lane / 16;
  const int ksl = K / kPWaves;                              // K slice of a wave
  const int steps = ksl / 64;                               // <= kPSteps
  const int n_begin = blockIdx.x * chan_per_wg;
  const int n_end = n_begin + chan_per_wg < N ? n_begin + chan_per_wg : N;

  for (int base = n_begin; base < n_end; base += kPTiles * 16) {
    // The scale of the output this thread will finish, requested before the weights: it comes from HBM and would
    // otherwise be waited for after everything else. (The empty asm below is a use on every path.)
    f16 sc;
    {
      const int q = (threadIdx.x / 256) % kPTiles, e = threadIdx.x % 256;
      const int gn = base + q * 16 + (e / 64) * 4 + e % 4;
      sc = scales[gn < n_end ? gn : n_end - 1];
    }
    // weights: all tiles of this pass, every step
    u32x4 wv[kPTiles][kPSteps];
#pragma unroll
    for (int q = 0; q < kPTiles; ++q) {
      int tile = base / 16 + q;
      const int last = (N + 15) / 16 - 1;
      tile = tile <= last ? tile : last;                    // past the end: re-read the last tile, unused
      const int8_t* blk = W + ((int64_t)tile * (K / 64) + (int64_t)wave * steps) * 1024 + lane * 16;
#pragma unroll
      for (int u = 0; u < kPSteps; ++u) {
        const int st = u < steps ? u : steps - 1;
        wv[q][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(blk + st * 1024));
      }
    }
    // this wave's activation slice: rows r16, k in [wave*ksl + u*64 + kg*16, +16)
    f16x8 av[kPSteps][2];
    {
      const f16* arow = A + (int64_t)(r16 < M ? r16 : 0) * K + (int64_t)wave * ksl + kg * 16;
#pragma unroll
      for (int u = 0; u < kPSteps; ++u) {
        const int st = u < steps ? u : steps - 1;
        av[u][0] = *reinterpret_cast<const f16x8*>(arow + st * 64);
        av[u][1] = *reinterpret_cast<const f16x8*>(arow + st * 64 + 8);
        if (r16 >= M) {
          av[u][0] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
          av[u][1] = av[u][0];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < kPTiles; ++q) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < kPSteps; ++u) {
        if (u < steps) {                                    // wave-uniform
          f16x8 w0, w1;
          cvt16(wv[q][u], w0, w1);
          // D[i = channel][j = activation row]: lane holds row j = lane%16, channels 4*(lane/16) + 0..3
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, av[u][0], acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, av[u][1], acc, 0, 0, 0);
        }
      }
      *reinterpret_cast<f32x4*>(red + ((q * kPWaves + wave) * 64 + lane) * 4) = acc;
    }
    asm volatile("" : "+v"(sc));
    __syncthreads();
    if (threadIdx.x < kPTiles * 256) {
      const int q = threadIdx.x / 256, e = threadIdx.x % 256;     // e = lane*4 + element of the accumulator
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < kPWaves; ++w) sum += red[(q * kPWaves + w) * 256 + e];
      const int l = e / 4;
      const int gm = l % 16;
      const int gn = base + q * 16 + (l / 16) * 4 + e % 4;
      if (gm < M && gn < n_end) C[(int64_t)gm * N + gn] = (f16)(sum * (float)sc);
    }
    __syncthreads();
  }
}

// 2 < M <= 128 (MB = 1, 2, 3, 4, 6 or 8 blocks of 16 activation rows; K any multiple of 64): persistent
// workgroups of 16 waves, each owning an equal contiguous range of at most 48 output channels, so the weights cross
// HBM once, in contiguous row segments. K is walked in chunks of KC = 256 (MB <= 4) or 128 (MB = 6, 8): an
// activation chunk is at most 32 KiB; with MB <= 2 and one or two channel tiles the chunks are 768 or 384 k long
// (mid_kc()). The raw int8 weight chunk [48][KC] and the activation chunk [MB*16][KC] fp16 are copied
// global -> LDS (global_load_lds, no registers) by different waves: waves 12..15 copy weights, four chunks ahead
// (five stages: three or four measured the same, seven and nine 5-10 % slower), waves 0..11 copy activations, two
// chunks ahead (three stages; L2 hits). A wave's outstanding-copy counter only sees its own copies, so each role
// waits with its own count and the workgroup barrier publishes both.
// Compute wave w < 12 owns channel tile w % 3 and, of every chunk, one unit of 64 k for one group of row blocks
// (four K units and all row blocks at KC = 256; two units and two groups of three or four row blocks at KC = 128;
// twelve units of one tile at KC = 768 and six of each of two tiles at KC = 384, where no wave is left over). It converts
// its 16 x 64 int8 weights to fp16 once per chunk (16 vector instructions) and multiplies them into its RB
// accumulators (2 * RB MFMAs). A SIMD issues one instruction at a time and a 16x16x32 MFMA hides only two vector
// instructions, so the conversions per MFMA set the pace: with one 16 x 16 tile per wave (every row-block wave
// converting the same weights, 8 to 10 instructions per MFMA) the kernel took 18.4 us at M = 64, N = 11008, K = 4096,
// this way 15.0 (22.6 -> 21.1 with the weights coming from HBM). Fragments are read back from LDS in 16-byte chunks
// permuted inside their row through the copies' source addresses (conflict-free). The K units of a tile are summed
// through LDS after the K loop, in a fixed order, and the tile is stored row by row (one wave, one row's channels).
// What a launch of this kernel costs besides the stream, from wall-clock stamps inside it (N = 11008, K = 4096,
// weights from HBM, median workgroup): 0.5-0.7 us to the first copies (a weight wave needs another 0.5-0.8 us to
// get its twelve issued), the first chunk there 2.4 us after the start, then a chunk every 0.45-0.5 us at 16 rows
// (6.0-6.3 TB/s: the HBM rate), 0.73 us at 64 (activations through L2); 0.3 us from the last chunk's barrier to the
// end of the loop and 0.5 us (16 rows) to 1.0 us (64, 128 rows) for the sum of the K units and the stores.
// With every CU fetching all of A the kernel moves M * 8 KiB per CU through L2: 29 us at M = 128 (the 128 x 128
// tile kernel, 86 tiles: 34), but 47 us at M = 256 with 64-k chunks (tile kernel: 37), so it stops at 128 rows.
constexpr int kMidWeightPolicy = 2;                         // nt: weights are read once (12.4 against 13.0 us at M = 16)
constexpr int kMidCh = 48;                                  // channels per workgroup (three tiles of 16)
constexpr int kMidAStages = 3, kMidWStages = 5;
constexpr int kMidCompute = 12;                             // compute waves: (channel tile, K unit, row-block group)
constexpr int kMidWWave0 = 12;                              // first of the four weight-copy waves
constexpr int kMidMaxM = 128;
// K per chunk. Sixteen rows leave LDS for longer chunks, and a workgroup with one or two channel tiles needs them:
// what a CU has in flight is four chunks of weights, 16 KiB with one tile of 256 k, too little to keep HBM busy
// (N = 4096, K = 11008, M = 16: 19.1 us), 48 KiB with 768 k.
constexpr int mid_kc(int mb, int nt) {
  return mb == 1 ? (nt == 1 ? 768 : nt == 2 ? 384 : 256) : mb == 2 ? (nt <= 2 ? 384 : 256) : mb <= 4 ? 256 : 128;
}
// s_waitcnt immediate (gfx9 encoding) that leaves `vm` vector-memory operations outstanding, LDS counter untouched
constexpr int wait_vm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | (0xF << 8); }

// position of 16-byte chunk c inside its row of CH chunks (an involution in c for a given row); rows of 256 and
// 512 bytes start at the same banks, so the row number itself spreads the chunks
template <int CH> __device__ __forceinline__ int mid_a_pos(int c, int row) {
  static_assert(CH % 16 == 0, "activation rows are whole bank cycles of 256 bytes");
  return (c & ~15) | ((c ^ row) & 15);
}
template <int CH> __device__ __forceinline__ int mid_w_pos(int c, int row) {
  if constexpr (CH % 16 == 0) return (c & ~15) | ((c ^ row) & 15);
  // rows of 128 or 384 bytes: consecutive rows start half a bank cycle apart, so pairs of rows share the low bits
  else return (c & ~7) | ((c ^ (row >> 1)) & 7);
}

// a branch on a wave's role (see the note at the copy slots)
#define HEXMI_EITHER(c) __builtin_expect((c), 1)
#define HEXMI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define HEXMI_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

// NT: channel tiles of 16 in use (a narrow matrix leaves a workgroup fewer than 48 channels): only their weight rows
// are copied. The compute waves of the other tiles run the same code on whatever their part of the stage holds
// (their sums are never stored): they are needed for the activation copies and the barriers, and a second code
// path for them costs the kernel registers it does not have.
// KC: K per chunk. K need not be a multiple of it: copies of a last, shorter chunk are
// clamped to the row and the 64-k units past K are multiplied as zeros.
// ZP: a zero point is subtracted from the widened weights (exact in fp16), as in w8a16_kernel above; per_tensor
// reads scale and zero point at index 0 for every channel (with or without ZP).
// TAIL: K % KC != 0 allowed. Without it the copies take a uniform chunk offset and the weights go unmasked, which
// the forms with more than 32 rows, short of registers and issue slots, run 5 % faster (M = 64: 17.0 against 18.0 us).
template <int MB, int NT = 3, int KC = mid_kc(MB, NT), bool ZP = false, bool TAIL = true>
__global__ __launch_bounds__(1024, (MB == 1 && NT == 2 && KC == 256) ? 8 : 4)
void w8a16_mid_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                      f16* __restrict__ C, int M, int N, int K, int chan_per_wg, int rotate,
                      const int8_t* __restrict__ zero_points = nullptr, int per_tensor = 0) {
  constexpr int KU = KC / 64;                               // 64-k units per chunk
  // channel-tile slots the twelve compute waves are laid out for: the tiles in use when their units and whole
  // groups of row blocks take all twelve, else three (the waves of a slot without channels run along)
  constexpr int TS = kMidCompute % (NT * KU) == 0 && MB % (kMidCompute / (NT * KU)) == 0 ? NT : 3;
  constexpr int RG = kMidCompute / TS / KU;                 // row-block groups
  static_assert(TS * KU * RG == kMidCompute && KC % 64 == 0, "every compute wave has a tile slot, a unit and a group");
  constexpr int RB = MB / RG;                               // row blocks per compute wave
  static_assert(MB % RG == 0 && RB >= 1 && RB <= 4, "row blocks split evenly over the groups");
  constexpr int ACH = KC / 8, WCH = KC / 16;                // 16-byte chunks per activation / weight row
  constexpr int NAC = MB * KC / 32, NWC = NT * 16 * KC / 1024;  // 1 KiB copies per chunk
  constexpr int ASL = (NAC + kMidCompute - 1) / kMidCompute, WSL = (NWC + 3) / 4;   // copy slots per wave
  constexpr int SL = ASL > WSL ? ASL : WSL;
  constexpr int WS = kMidWStages;
  __shared__ __attribute__((aligned(16))) f16 a_s[kMidAStages][MB * 16 * KC];
  __shared__ __attribute__((aligned(16))) int8_t w_s[WS][NT * 16 * KC];

  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int r16 = lane % 16, kg = lane / 16;
  const int n_begin = blockIdx.x * chan_per_wg;
  const int n_end = n_begin + chan_per_wg < N ? n_begin + chan_per_wg : N;
  const int n_chunks = (K + KC - 1) / KC;                   // TAIL: the last one may be short (K % 16 == 0)
  // Workgroup b walks K from chunk b % n_chunks on and wraps round. With every workgroup at the same k at the
  // same time, all the addresses in flight on the chip agree in their low bits when the weight rows are a power of
  // two long, and the memory channels those bits select take the whole load (N = 8192, M = 16: 20.9 us at
  // K = 8192, 14.2 at 7936, 15.0 at 8320). The order of a channel's sum so depends on the workgroup it falls in.
  // Not with two workgroups per CU at a time (rotate = 0): there it costs 4-7 %.
  const int rot = rotate ? (int)(blockIdx.x % (unsigned)n_chunks) : 0;
  auto k_chunk = [&](int chunk) __attribute__((always_inline)) {
    return chunk + rot < n_chunks ? chunk + rot : chunk + rot - n_chunks;
  };
  const bool computes = wave < kMidCompute;                 // also copies activations
  const bool copies_w = wave >= kMidWWave0;
  // The channel scales come from HBM: requested first (older than every copy of this wave, so the counted waits
  // below see them finished) they are there when the K loop ends; requested after it they are a memory latency
  // on the way out.
  f16 my_scale = (f16)0.0f;
  if (threadIdx.x < kMidCh) {
    const int gn = n_begin + (int)threadIdx.x;
    my_scale = scales[per_tensor ? 0 : (gn < n_end ? gn : n_end - 1)];
  }

  // ---- copy slots: every copy moves 1 KiB, 64 consecutive 16-byte pieces of the stage (a row may end inside it);
  //      lane positions are permuted inside a row (see the fragment side). Slots past the last real copy repeat one
  //      (same bytes, rewritten).
  const char* slot_src[SL];                                 // source of this lane for chunk 0
  int slot_dst[SL];                                         // byte offset of the copy inside its stage
  int slot_lim[SL];                                         // largest chunk offset that keeps this lane inside its row
  // Before the loop, every piece of code that only one role runs is an `if` of its own marked as expected, never an
  // else branch: the compiler places an else branch it takes for the unlikely one behind the loop, and a jump into
  // code not yet fetched costs a kernel that has just started about half a microsecond (the weight waves' slots,
  // their first copies and their first wait were three such jumps; 1-2 % of the kernel at 16 rows). The slots of
  // the other role stay unset: nothing reads them.
  if (HEXMI_EITHER(copies_w)) {
#pragma unroll
    for (int j = 0; j < WSL; ++j) {
      const int t = (j * 4 + (wave - kMidWWave0)) % NWC;
      const int f = t * 64 + lane;                          // 16-byte piece of the stage: 64 per copy
      const int row = f / WCH;
      const int src_c = mid_w_pos<WCH>(f % WCH, row);       // the chunk that belongs at this position
      const int n = n_begin + row < n_end ? n_begin + row : n_end - 1;
      slot_src[j] = reinterpret_cast<const char*>(W + (int64_t)n * K) + src_c * 16;
      slot_dst[j] = t * 1024;
      slot_lim[j] = K - 16 - src_c * 16;
    }
  }
  if (HEXMI_EITHER(computes)) {
#pragma unroll
    for (int j = 0; j < ASL; ++j) {
      const int i = (j * kMidCompute + wave) % NAC;
      const int f = i * 64 + lane;
      const int row = f / ACH;
      const int src_c = mid_a_pos<ACH>(f % ACH, row);
      slot_src[j] = reinterpret_cast<const char*>(A + (int64_t)(row < M ? row : M - 1) * K) + src_c * 16;
      slot_dst[j] = i * 1024;
      slot_lim[j] = K * 2 - 16 - src_c * 16;
    }
  }
  // chunk indices past the end repeat the last chunk (copied, never read): every chunk issues the same copies
  // LDS stages by byte address (a stage index counted at run time must not turn into generic pointers)
  typedef __attribute__((address_space(3))) char* lds_ptr;
  const unsigned a_lds = (unsigned)(size_t)(lds_ptr)(&a_s[0][0]);
  const unsigned w_lds = (unsigned)(size_t)(lds_ptr)(&w_s[0][0]);
  constexpr unsigned kAStage = MB * 16 * KC * 2, kWStage = NT * 16 * KC;
  // A lane whose piece of the last chunk lies past K fetches the last 16 bytes of its row instead (never
  // multiplied: see the mask in multiply()).
  auto issue_a = [&](int chunk, unsigned dst) __attribute__((always_inline)) {
    const int ck = k_chunk(chunk < n_chunks ? chunk : n_chunks - 1);
#pragma unroll
    for (int j = 0; j < ASL; ++j) {
      const int off = ck * (KC * 2);
      const char* src = TAIL ? slot_src[j] + (off < slot_lim[j] ? off : slot_lim[j]) : slot_src[j] + (int64_t)ck * (KC * 2);
      __builtin_amdgcn_global_load_lds(HEXMI_GLB(src), (lds_ptr)(size_t)(dst + slot_dst[j]), 16, 0, 0);
    }
  };
  auto issue_w = [&](int chunk, unsigned dst) __attribute__((always_inline)) {
    const int ck = k_chunk(chunk < n_chunks ? chunk : n_chunks - 1);
#pragma unroll
    for (int j = 0; j < WSL; ++j) {
      const int off = ck * KC;
      const char* src = TAIL ? slot_src[j] + (off < slot_lim[j] ? off : slot_lim[j]) : slot_src[j] + (int64_t)ck * KC;
      __builtin_amdgcn_global_load_lds(HEXMI_GLB(src), (lds_ptr)(size_t)(dst + slot_dst[j]), 16, 0, kMidWeightPolicy);
    }
  };

  // ---- fragment side: compute wave w owns channel tile nt = w % 3, K unit ku and row-block group rg
  const int nt = wave % TS, ku = (wave / TS) % KU, rg = (wave / TS) / KU;
  // A chunk's position depends on the row only through its low four bits, so row block rb of the group is a
  // constant 16 * KC * 2 * rb bytes further: an immediate offset of the read, not a register.
  int w_off, a_off[2];
  {
    const int wrow = (nt < NT ? nt : 0) * 16 + r16;          // a tile without channels reads tile 0's part of the stage
    w_off = wrow * KC + mid_w_pos<WCH>(ku * 4 + kg, wrow) * 16;
    const int arow = rg * RB * 16 + r16;
#pragma unroll
    for (int h = 0; h < 2; ++h) a_off[h] = arow * KC * 2 + mid_a_pos<ACH>(ku * 8 + kg * 2 + h, arow) * 16;
  }
  static_assert((RB - 1) * 16 * KC * 2 < 65536, "row-block offsets fit the read's immediate");
  f32x4 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
  f16 zp_h = (f16)0.0f;                                     // ZP: set in the prologue
  // The fragment reads are written as inline assembly: the compiler cannot tell which stage an in-flight
  // global_load_lds writes and would make every LDS read wait for all of them (vmcnt(0)), which undoes the
  // pipelining. The waits this kernel needs are the explicit ones around the barrier.
  // Fragments are double-buffered in registers: the reads of chunk u+1 are issued before the arithmetic of chunk u
  // and waited for at the top of the next round, so the LDS latency passes under the conversions and MFMAs. The wait
  // statement names every fragment register as modified: nothing that uses one can be scheduled above it.
  struct Frags { u32x4 raw, a0[RB], a1[RB]; };
  auto read_frags = [&](Frags& f, unsigned a_base, unsigned w_base) __attribute__((always_inline)) {
    asm volatile("ds_read_b128 %0, %1" : "=&v"(f.raw) : "v"(w_base + w_off) : "memory");
    const unsigned a_at0 = a_base + a_off[0], a_at1 = a_base + a_off[1];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(f.a0[rb]) : "v"(a_at0), "n"(rb * 16 * KC * 2) : "memory");
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(f.a1[rb]) : "v"(a_at1), "n"(rb * 16 * KC * 2) : "memory");
    }
  };
  auto wait_frags = [&](Frags& f) __attribute__((always_inline)) {
    if constexpr (RB == 4)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.raw), "+v"(f.a0[0]), "+v"(f.a1[0]), "+v"(f.a0[1]), "+v"(f.a1[1]),
                   "+v"(f.a0[2]), "+v"(f.a1[2]), "+v"(f.a0[3]), "+v"(f.a1[3]) :: "memory");
    else if constexpr (RB == 3)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.raw), "+v"(f.a0[0]), "+v"(f.a1[0]), "+v"(f.a0[1]), "+v"(f.a1[1]),
                   "+v"(f.a0[2]), "+v"(f.a1[2]) :: "memory");
    else if constexpr (RB == 2)
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.raw), "+v"(f.a0[0]), "+v"(f.a1[0]), "+v"(f.a0[1]), "+v"(f.a1[1]) :: "memory");
    else
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f.raw), "+v"(f.a0[0]), "+v"(f.a1[0]) :: "memory");
  };
  auto multiply = [&](const Frags& f, int chunk) __attribute__((always_inline)) {
    f16x8 w0, w1;
    // a lane's sixteen weights past the end of K (K % 16 == 0) are the bytes its copy was clamped to: they count as
    // zeros (and so does their zero point)
    const unsigned keep = !TAIL || k_chunk(chunk) * KC + (ku * 4 + kg) * 16 < K ? 0xffffffffu : 0u;
    if constexpr (TAIL) {
      const u32x4 raw = {f.raw[0] & keep, f.raw[1] & keep, f.raw[2] & keep, f.raw[3] & keep};
      cvt16(raw, w0, w1);                                   // converted once, used for every row block
    } else {
      cvt16(f.raw, w0, w1);
    }
    if constexpr (ZP) {
      const f16 z = __builtin_bit_cast(f16, (unsigned short)(__builtin_bit_cast(unsigned short, zp_h) & keep));
      w0 -= z;                                              // exact: integers of magnitude <= 255
      w1 -= z;
    }
    // D[i = channel][j = activation row]: lane holds row j = lane%16, channels 4*(lane/16) + 0..3
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, __builtin_bit_cast(f16x8, f.a0[rb]), acc[rb], 0, 0, 0);
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, __builtin_bit_cast(f16x8, f.a1[rb]), acc[rb], 0, 0, 0);
  };
  // prologue: activations of chunks 0, 1; weights of chunks 0 .. 3
  if (HEXMI_EITHER(copies_w)) {
#pragma unroll
    for (int i = 0; i < WS - 1; ++i) issue_w(i, w_lds + i * kWStage);
  }
  if (HEXMI_EITHER(computes)) {
    issue_a(0, a_lds);
    issue_a(1, a_lds + kAStage);
    if constexpr (ZP) {
      // The zero point of the channel whose weights this lane converts (lane % 16 of the wave's tile), requested
      // behind the first activation copies and waited for, with them, before the first barrier: it comes from HBM
      // like the first weights everybody waits for there, and once it is a plain register value the compiler has no
      // load to wait for inside the loop, where its wait would cover every copy in flight in every round. (Weight
      // waves must not take part: the same wait would cover all their copies.)
      const int gn = n_begin + (nt < NT ? nt : 0) * 16 + r16;
      int my_zp = zero_points[per_tensor ? 0 : (gn < n_end ? gn : n_end - 1)];
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(my_zp) :: "memory");
      zp_h = (f16)(float)my_zp;
    }
  }
  // Round u: chunk u+1 has landed for every wave after the barrier (each role waited for its own copies of it) and
  // every wave has the fragments of chunk u in registers, so the stages of chunk u are free: the copies of chunk
  // u+3 (activations) and u+WS (weights) go there. Then the fragments of chunk u+1 are requested and chunk u is
  // multiplied. Round -1 (before the loop) fetches the fragments of chunk 0.
  if (HEXMI_EITHER(copies_w)) __builtin_amdgcn_s_waitcnt(wait_vm((WS - 2) * WSL));   // chunk 0 landed
  if (HEXMI_EITHER(computes)) __builtin_amdgcn_s_waitcnt(wait_vm(ASL));
  __builtin_amdgcn_s_barrier();
  Frags fa, fb;
  if (HEXMI_EITHER(copies_w)) issue_w(WS - 1, w_lds + (WS - 1) * kWStage);
  if (HEXMI_EITHER(computes)) {
    issue_a(2, a_lds + 2 * kAStage);
    read_frags(fa, a_lds, w_lds);
  }
  // The loop is unrolled by two only (the two register buffers alternate); the LDS stages are counted at run time
  // in scalar registers. A kernel's instruction cache starts cold and a jump to code not yet fetched costs about
  // half a microsecond here (measured: the exit from the middle of a long unrolled loop to the code behind it), so
  // the loop is short, every round after the first two runs from the cache, and the way out is a fall through: an
  // odd last chunk is a copy of the round placed behind the loop, and the sum of the K units follows it in line.
  // A round with `togo` rounds to go (itself included) copies activations only if togo > 3 and weights only if
  // togo > 5: nothing is fetched twice and nothing is in flight when the K loop ends. Its waits leave fewer copies
  // outstanding accordingly; the count of an s_waitcnt is an immediate, so each is a short ladder of uniform
  // branches with nothing but the wait inside.
  // Registers with a read in flight must never be moved: apart from those ladders a round's body is straight-line
  // code, and the buffer whose reads cross the back edge is waited for first. The fragment reads of a round with
  // nothing behind it fetch a stage nobody multiplies: the same instructions every round.
  unsigned sa = a_lds, sw = w_lds;                           // stages of the current chunk, as LDS addresses
  auto round = [&](int chunk, Frags& cur, Frags& nxt, bool reads) __attribute__((always_inline)) {
    const int togo = n_chunks - chunk;
    if (computes) {
      wait_frags(cur);                                      // fragments of this chunk are in registers
      // own copies of chunk + 1 have landed; those of chunk + 2, if there is one, may be outstanding
      if (togo >= 3) __builtin_amdgcn_s_waitcnt(wait_vm(ASL));
      else __builtin_amdgcn_s_waitcnt(wait_vm(0));
    } else if (copies_w) {
      // chunk + 1 has landed; up to three younger chunks may be outstanding
      if (togo >= 5) __builtin_amdgcn_s_waitcnt(wait_vm(3 * WSL));
      else if (togo == 4) __builtin_amdgcn_s_waitcnt(wait_vm(2 * WSL));
      else if (togo == 3) __builtin_amdgcn_s_waitcnt(wait_vm(WSL));
      else __builtin_amdgcn_s_waitcnt(wait_vm(0));
    }
    // A bare s_barrier: __syncthreads() would add a wait for every outstanding copy and undo the pipelining.
    __builtin_amdgcn_s_barrier();
    const unsigned sa1 = sa + kAStage == a_lds + kMidAStages * kAStage ? a_lds : sa + kAStage;
    const unsigned sw1 = sw + kWStage == w_lds + WS * kWStage ? w_lds : sw + kWStage;
    if (computes) {
      if (togo > 3) issue_a(chunk + 3, sa);
      if (reads) read_frags(nxt, sa1, sw1);
      // With one row block the round is short and the order of its few instructions shows: the next chunk's reads
      // go out whole before the first MFMA (2-3 % at sixteen rows under graph replay). With more row blocks the
      // compiler's own interleaving is as good or better.
      if constexpr (MB == 1) __builtin_amdgcn_sched_barrier(0);
      multiply(cur, chunk);
    } else if (copies_w) {
      if (togo > WS) issue_w(chunk + WS, sw);
    }
    sa = sa1;
    sw = sw1;
  };
  static_assert(kMidAStages == 3 && kMidWStages == 5, "the waits of a round are written for these depths");
  int chunk = 0;
  for (; chunk + 2 <= n_chunks; chunk += 2) {
    round(chunk, fa, fb, true);
    round(chunk + 1, fb, fa, true);
    if (computes) wait_frags(fa);
  }
  if (chunk < n_chunks) round(chunk, fa, fb, false);

  // ---- the K units of every tile are summed through LDS and the tile goes out in rows: partial tiles as
  //      [unit][row][48 channels] fp32 in the activation stages, then compute wave w adds up rows w, w + 12, ... in
  //      the fixed order unit 0 + 1 + ..., lane = channel, scales them and stores them: a store covers one row's
  //      channels side by side (a lane's own four outputs are 2-byte pieces of 16 different rows).
  // After the last round's barrier every wave holds its last fragments in registers and no copy is in flight, so
  // the stages are free. Only with fewer than three chunks (activations) or five (weights) can a copy of the
  // prologue, which then repeats the last chunk, still be on its way: the compute waves then wait for theirs and
  // meet once more before the stages are written, and the copy waves, whose stages nothing below touches, wait for
  // theirs alone before they end (the LDS is released when the last wave has ended). The barriers are bare
  // s_barriers with the waits each role needs written out.
  constexpr int ROWS = MB * 16;
  float* red = reinterpret_cast<float*>(&a_s[0][0]);
  // rows of 52 floats: a wave's 16 rows of four-float pieces then fall on 16 different groups of four banks
  // (rows of 48 floats put four rows on every group)
  constexpr int RS = kMidCh + 4;
  float* sc_s = red + KU * ROWS * RS;                       // the channel scales of this workgroup, as fp32
  static_assert((KU * ROWS + 1) * RS * 4 <= kMidAStages * ROWS * KC * 2, "the partial tiles fit the activation stages");
  if (n_chunks < kMidAStages) {
    if (computes) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  }
  // the scale is first used here: without this the compiler converts it to fp32 where it is loaded and makes wave 0
  // wait for an HBM access before its first copies
  asm volatile("" : "+v"(my_scale));
  if (computes) {
    if (threadIdx.x < kMidCh) sc_s[threadIdx.x] = (float)my_scale;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int row = (rg * RB + rb) * 16 + r16;
      *reinterpret_cast<f32x4*>(red + ((ku * ROWS + row) * RS + nt * 16 + kg * 4)) = acc[rb];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (!computes) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }
  const int rows = M < ROWS ? M : ROWS;
  if (lane < n_end - n_begin) {                              // a wave writes one row's channels side by side
    const float scale = sc_s[lane];
    constexpr int PASSES = (ROWS + kMidCompute - 1) / kMidCompute;
    float part[PASSES][KU];
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {                       // all reads first: one LDS latency, not one per row
      const int row = wave + i * kMidCompute < ROWS ? wave + i * kMidCompute : ROWS - 1;
#pragma unroll
      for (int q = 0; q < KU; ++q) part[i][q] = red[(q * ROWS + row) * RS + lane];
    }
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
      const int row = wave + i * kMidCompute;
      float sum = part[i][0];
#pragma unroll
      for (int q = 1; q < KU; ++q) sum += part[i][q];
      if (row < rows) C[(int64_t)row * N + n_begin + lane] = (f16)(sum * scale);
    }
  }
}

#undef HEXMI_EITHER
#undef HEXMI_LDS
#undef HEXMI_GLB

// One or two activation rows (decode): no matrix cores. A wave owns RPW consecutive output channels and reads
// each 4 KiB-aligned weight row with fully contiguous 16-byte loads (lane i takes bytes [1024*j + 16*i, +16) of
// the row for j = 0..K/1024), all RPW rows in flight at once; the activations a lane needs (the same k for every
// row) sit in registers as fp16 pairs. Products are v_dot2_f32_f16 (two exact fp16 products added into an fp32
// accumulator), the 64 lane partials are summed with a butterfly, and lane 0 applies the channel scale.
// NW waves per workgroup share the activation rows through LDS.
// ZP / per_tensor: as in the kernels above (the zero point is subtracted from the widened weights).
template <int MR, int RPW, int KJ, int NW = 4, bool ZP = false>   // KJ = K / 1024: 16-byte loads per lane per row
__global__ __launch_bounds__(NW * 64)
void w8a16_gemv_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                       f16* __restrict__ C, int M, int N, int K, const int8_t* __restrict__ zero_points = nullptr,
                       int per_tensor = 0) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n0 = (blockIdx.x * NW + wave) * RPW;           // may lie past N in the last workgroup: loads clamp, stores check

  // the channel scales first: they come from HBM and would otherwise be waited for after everything else
  f16 sc[RPW], zp[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int at = per_tensor ? 0 : (n0 + r < N ? n0 + r : N - 1);
    sc[r] = scales[at];
    zp[r] = (f16)0.0f;
    if constexpr (ZP) zp[r] = (f16)(float)zero_points[at];
  }
  // activations: lane needs k in [1024*j + 16*lane, +16) for every j. The four waves of the workgroup need the same
  // rows, so each fetches a quarter of them (requested before the weights: their wait then leaves the weight loads in
  // flight) and all read their fragments back from LDS.
  __shared__ __attribute__((aligned(16))) f16 a_lds[MR][KJ * 1024];
  constexpr int kAChunks = (KJ * 128 + NW * 64 - 1) / (NW * 64);
  f16x8 a_in[MR][kAChunks];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const f16* arow = A + (int64_t)(m < M ? m : 0) * K;
#pragma unroll
    for (int c = 0; c < kAChunks; ++c) {
      const int chunk = c * (NW * 64) + threadIdx.x;
      a_in[m][c] = *reinterpret_cast<const f16x8*>(arow + (chunk < KJ * 128 ? chunk : 0) * 8);
    }
  }
  u32x4 wv[RPW][KJ];
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const int n = n0 + r < N ? n0 + r : N - 1;
    const int8_t* wrow = W + (int64_t)n * K + lane * 16;
#pragma unroll
    for (int j = 0; j < KJ; ++j) wv[r][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + j * 1024));
  }
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int c = 0; c < kAChunks; ++c) {
      const int chunk = c * (NW * 64) + threadIdx.x;
      if (chunk < KJ * 128) *reinterpret_cast<f16x8*>(&a_lds[m][chunk * 8]) = a_in[m][c];
    }
  __syncthreads();
  f16x8 av[MR][KJ][2];
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int j = 0; j < KJ; ++j) {
      av[m][j][0] = *reinterpret_cast<const f16x8*>(&a_lds[m][j * 1024 + lane * 16]);
      av[m][j][1] = *reinterpret_cast<const f16x8*>(&a_lds[m][j * 1024 + lane * 16 + 8]);
    }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.0f;
#pragma unroll
    for (int j = 0; j < KJ; ++j) {
      f16x8 w0, w1;
      cvt16(wv[r][j], w0, w1);
      if constexpr (ZP) {
        w0 -= zp[r];
        w1 -= zp[r];
      }
#pragma unroll
      for (int m = 0; m < MR; ++m) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[m] = __builtin_amdgcn_fdot2(f16x2{w0[2 * e], w0[2 * e + 1]}, f16x2{av[m][j][0][2 * e], av[m][j][0][2 * e + 1]},
                                          acc[m], false);
          acc[m] = __builtin_amdgcn_fdot2(f16x2{w1[2 * e], w1[2 * e + 1]}, f16x2{av[m][j][1][2 * e], av[m][j][1][2 * e + 1]},
                                          acc[m], false);
        }
      }
    }
    const int n = n0 + r;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const float tot = wave_sum(acc[m]);
      if (lane == 0 && n < N && m < M) C[(int64_t)m * N + n] = (f16)(tot * (float)sc[r]);
    }
  }
}

// The same decode kernel for any K that is a multiple of 16 (up to NJ KiB per row): lane i takes the 16-byte pieces
// i, i + 64, ... of the row, the last round masked where the row has ended (zero weights). One channel per wave; the
// activation rows are staged in LDS once per workgroup and read back piece by piece, so the
// registers hold the row's weight loads (all in flight at once) and little else. Sixteen waves per workgroup (N = 4096,
// K = 11008: 11.5 us against 11.9 with eight and 12.0 with four: fewer workgroups stage the activation row).
template <int MR, int NJ, int NW = 16, bool ZP = false>
__global__ __launch_bounds__(NW * 64)
void w8a16_gemv_any_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                           f16* __restrict__ C, int M, int N, int K, const int8_t* __restrict__ zero_points = nullptr,
                           int per_tensor = 0) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = blockIdx.x * NW + wave;                     // may lie past N in the last workgroup: loads clamp
  const f16 sc = scales[per_tensor ? 0 : (n < N ? n : N - 1)];
  f16 zp = (f16)0.0f;
  if constexpr (ZP) zp = (f16)(float)zero_points[per_tensor ? 0 : (n < N ? n : N - 1)];
  const int pieces = K / 16;                                // 16-byte pieces of a weight row
  u32x4 wv[NJ];
  {
    const int8_t* wrow = W + (int64_t)(n < N ? n : N - 1) * K;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int pc = j * 64 + lane;
      wv[j] = u32x4{0u, 0u, 0u, 0u};
      if (pc < pieces) wv[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + pc * 16));
    }
  }
  __shared__ __attribute__((aligned(16))) f16 a_lds[MR][NJ * 1024];
  for (int m = 0; m < MR; ++m) {
    const f16* arow = A + (int64_t)(m < M ? m : 0) * K;
    for (int c = threadIdx.x; c < K / 8; c += NW * 64)
      *reinterpret_cast<f16x8*>(&a_lds[m][c * 8]) = *reinterpret_cast<const f16x8*>(arow + c * 8);
  }
  __syncthreads();
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.0f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int pc = j * 64 + lane;
    if (j * 64 < pieces) {                                  // wave-uniform: rounds past the row do nothing
      f16x8 w0, w1;
      cvt16(wv[j], w0, w1);
      if constexpr (ZP) {
        const f16 z = pc < pieces ? zp : (f16)0.0f;         // a masked lane's weights stay zero
        w0 -= z;
        w1 -= z;
      }
      const int at = (pc < pieces ? pc : 0) * 16;           // masked lanes hold zero weights; any valid address
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const f16x8 a0 = *reinterpret_cast<const f16x8*>(&a_lds[m][at]);
        const f16x8 a1 = *reinterpret_cast<const f16x8*>(&a_lds[m][at + 8]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[m] = __builtin_amdgcn_fdot2(f16x2{w0[2 * e], w0[2 * e + 1]}, f16x2{a0[2 * e], a0[2 * e + 1]}, acc[m], false);
          acc[m] = __builtin_amdgcn_fdot2(f16x2{w1[2 * e], w1[2 * e + 1]}, f16x2{a1[2 * e], a1[2 * e + 1]}, acc[m], false);
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const float tot = wave_sum(acc[m]);
    if (lane == 0 && n < N && m < M) C[(int64_t)m * N + n] = (f16)(tot * (float)sc);
  }
}

// One-time re-layout of int8 weights [N, K] into fragment-major order for the small-M kernels (the analogue of
// the reference's constant-weight block linearisation, qcom_hexagon_backend/lib/Transforms/
// PreprocessWeightsForHMXPass.cpp:39-117): tiles of 16 channels x 64 k, tile (t, s) at byte
// ((t * K/64) + s) * 1024, inside it lane l = g*16 + r holds the 16 bytes W[16t + r][64s + 16g .. +16).
// Channels past N (the last tile) are zero. One thread per 16-byte chunk of the output.
__global__ __launch_bounds__(256)
void pack_w8_kernel(const int8_t* __restrict__ W, int8_t* __restrict__ Wp, int64_t N, int64_t K, int64_t chunks) {
  const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (o >= chunks) return;
  const int lane = (int)(o % 64);
  const int64_t blk = o / 64;                                // t * K/64 + s
  const int64_t t = blk / (K / 64), sidx = blk % (K / 64);
  const int64_t row = t * 16 + lane % 16;
  const int64_t k = sidx * 64 + (lane / 16) * 16;
  u32x4 v = {0u, 0u, 0u, 0u};
  if (row < N) v = *reinterpret_cast<const u32x4*>(W + row * K + k);
  *reinterpret_cast<u32x4*>(Wp + o * 16) = v;
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

__global__ __launch_bounds__(256)
void dequant_ex_kernel(const int8_t* __restrict__ W, const f16* __restrict__ scales, const int8_t* __restrict__ zero_points,
                       int per_tensor, float* __restrict__ out, int64_t N, int64_t K) {
  const int64_t total = N * K;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t n = per_tensor ? 0 : i / K;
    const float zp = zero_points ? (float)zero_points[n] : 0.0f;
    out[i] = ((float)W[i] - zp) * (float)scales[n];    // the difference is an exact integer, then one fp32 multiply
  }
}

// Any K and any alignment (the shapes the 16-byte-load kernels above do not take): one wave per output channel
// and block of MR activation rows, lanes stride over k, fp32 multiply-add of the exact int8 -> fp32 and
// fp16 -> fp32 values, butterfly sum, the channel scale on the finished sum as everywhere else.
template <int MR>
__global__ __launch_bounds__(256)
void w8a16_generic_kernel(const f16* __restrict__ A, const int8_t* __restrict__ W, const f16* __restrict__ scales,
                          f16* __restrict__ C, int M, int N, int K, const int8_t* __restrict__ zero_points = nullptr,
                          int per_tensor = 0) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n = blockIdx.x * 4 + wave;
  const int m0 = blockIdx.y * MR;
  if (n >= N) return;
  const int8_t* wrow = W + (int64_t)n * K;
  float acc[MR];
#pragma unroll
  for (int m = 0; m < MR; ++m) acc[m] = 0.0f;
  const float zp = zero_points ? (float)zero_points[per_tensor ? 0 : n] : 0.0f;
  for (int k = lane; k < K; k += kWave) {
    const float w = (float)wrow[k] - zp;
#pragma unroll
    for (int m = 0; m < MR; ++m)
      if (m0 + m < M) acc[m] = fmaf((float)A[(int64_t)(m0 + m) * K + k], w, acc[m]);
  }
  const float sc = (float)scales[per_tensor ? 0 : n];
#pragma unroll
  for (int m = 0; m < MR; ++m) {
    const float tot = wave_sum(acc[m]);
    if (lane == 0 && m0 + m < M) C[(int64_t)(m0 + m) * N + n] = (f16)(tot * sc);
  }
}

template <int MT>
int launch_pass(const f16* A, const int8_t* W, const f16* s, f16* C, int M, int N, int K, int m_base,
                hipStream_t st) {
  const int n_tiles = (N + 15) / 16;
  hipLaunchKernelGGL((w8a16_kernel<MT>), dim3(n_tiles), dim3(kThreads), 0, st, A, W, s, C, M, N, K, m_base);
  return launch_status();
}
template <int MT>
int launch_pass_zp(const f16* A, const int8_t* W, const f16* s, f16* C, int M, int N, int K, int m_base,
                   const int8_t* zp, int per_tensor, hipStream_t st) {
  const int n_tiles = (N + 15) / 16;
  hipLaunchKernelGGL((w8a16_kernel<MT, true>), dim3(n_tiles), dim3(kThreads), 0, st, A, W, s, C, M, N, K, m_base, zp,
                     per_tensor);
  return launch_status();
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

namespace {
// hexmi_gemm_w8a16 (zp == nullptr, pt == 0) and hexmi_gemm_w8a16_ex: one choice of kernels for both. The decode
// kernels and the chunked kernel have a zero-point instantiation; the 128 x 128 tile kernel does not, so more than
// 128 rows with a zero point or a per-tensor scale run the chunked kernel in passes of 128 rows.
int gemm_w8a16_any(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* W, const void* scales,
                   const int8_t* zp, int pt, void* C, hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!C || (K > 0 && (!A || !W || !scales))) return HEXMI_EINVAL;
  if (M > 0x7fffffff || N > 0x7fffffff - 16 || K > 0x7fffffff) return HEXMI_ENOTSUP;
  hipStream_t st = as_stream(stream);
  const f16* a = static_cast<const f16*>(A);
  const f16* s = static_cast<const f16*>(scales);
  f16* c = static_cast<f16*>(C);
  begin_call();
  if (K == 0) return fill_zero_2d(C, M, N, N, 2, st);      // an empty sum
  // two rows over a long K and at least 16 channels per CU go faster through the chunked kernel further down
  // (N = 4096, K = 11008: 11.2 against 12.9 us; N = K = 8192: 14.1 against 18.0)
  const bool chunked_pair = M == 2 && K >= 8192 && K % 64 == 0 && N >= 4096 && aligned_to(A, 16) && aligned_to(W, 16);
  if (M <= 2 && !chunked_pair && K % 16 == 0 && K <= 16384 && K != 1024 && K != 2048 && K != 4096 && K != 8192 && aligned_to(A, 16) &&
      aligned_to(W, 16)) {
    // any other row length: the masked form of the same kernel, instantiated per KiB of row
    const unsigned blocks = (unsigned)((N + 15) / 16);
    const int nj = (int)((K + 1023) / 1024);
#define HEXMI_GEMV_ANY(MR, NJ) { if (zp) hipLaunchKernelGGL((w8a16_gemv_any_kernel<MR, NJ, 16, true>), dim3(blocks), dim3(1024), 0, st, a, W, s, c, (int)M, (int)N, (int)K, zp, pt); \
    else hipLaunchKernelGGL((w8a16_gemv_any_kernel<MR, NJ, 16, false>), dim3(blocks), dim3(1024), 0, st, a, W, s, c, (int)M, (int)N, (int)K, zp, pt); }
#define HEXMI_GEMV_ANY_NJ(MR) switch (nj) { \
    case 1: HEXMI_GEMV_ANY(MR, 1); break; case 2: HEXMI_GEMV_ANY(MR, 2); break; case 3: HEXMI_GEMV_ANY(MR, 3); break; \
    case 4: HEXMI_GEMV_ANY(MR, 4); break; case 5: HEXMI_GEMV_ANY(MR, 5); break; case 6: HEXMI_GEMV_ANY(MR, 6); break; \
    case 7: HEXMI_GEMV_ANY(MR, 7); break; case 8: HEXMI_GEMV_ANY(MR, 8); break; case 9: HEXMI_GEMV_ANY(MR, 9); break; \
    case 10: HEXMI_GEMV_ANY(MR, 10); break; case 11: HEXMI_GEMV_ANY(MR, 11); break; case 12: HEXMI_GEMV_ANY(MR, 12); break; \
    case 13: HEXMI_GEMV_ANY(MR, 13); break; case 14: HEXMI_GEMV_ANY(MR, 14); break; case 15: HEXMI_GEMV_ANY(MR, 15); break; \
    default: HEXMI_GEMV_ANY(MR, 16); break; }
    if (M == 1) { HEXMI_GEMV_ANY_NJ(1) } else { HEXMI_GEMV_ANY_NJ(2) }
#undef HEXMI_GEMV_ANY_NJ
#undef HEXMI_GEMV_ANY
    return launch_status();
  }
  // the fast kernels copy 16 bytes of a weight row per lane: K % 16 == 0 and aligned bases; other shapes take the
  // generic one. (K % 64 != 0 runs the chunked kernel, in passes of 128 rows where the tile kernel does not apply.)
  const bool tile_kernel = !zp && !pt && M > 64 && K % 64 == 0 && N % 8 == 0 && aligned_to(C, 16) && aligned_to(scales, 8);
  if (K % 16 != 0 || !aligned_to(A, 16) || !aligned_to(W, 16) || (K % 64 != 0 && K > (1 << 29))) {
    // Enough output for it: 128x128 tiles on the matrix cores, the slabs staged through registers at any alignment
    // (N = 11008, K = 4040: M = 64 1.43 -> 0.14 ms, M = 1024 22.5 -> 0.23 ms). With few tiles that kernel waits out a
    // memory latency per slab (about 110 us at K = 4040 whatever the rows), and the kernel below, a wave per channel
    // with lanes striding over k, is ahead while M * N stays small (M = 16: 76 us at N = 4096, 371 at N = 11008).
    if (M > 8 && M * N >= 98304) return gemm_w8a16_any_shape(M, N, K, a, W, s, zp, pt, c, st);
    constexpr int MR = 4;
    const int64_t gy = (M + MR - 1) / MR;
    if (gy > 65535) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL(w8a16_generic_kernel<MR>, dim3((unsigned)((N + 3) / 4), (unsigned)gy), dim3(256), 0, st, a, W, s,
                       c, (int)M, (int)N, (int)K, zp, pt);
    return launch_status();
  }
  if (M <= 2 && !chunked_pair && (K == 1024 || K == 2048 || K == 4096 || K == 8192)) {
    // one channel per wave, eight waves per workgroup: measured against two and four channels per wave and
    // workgroups of two, four and sixteen waves at N = 11008, K = 4096 (0.60 of the HBM figure against 0.57 for two
    // channels x four waves on the same box)
    constexpr int RPW = 1, NW = 8;
    const unsigned blocks = (unsigned)((N + NW * RPW - 1) / (NW * RPW));
#define HEXMI_GEMV(MR, KJ) { if (zp) hipLaunchKernelGGL((w8a16_gemv_kernel<MR, RPW, KJ, NW, true>), dim3(blocks), dim3(NW * 64), 0, st, a, W, s, c, (int)M, (int)N, (int)K, zp, pt); \
    else hipLaunchKernelGGL((w8a16_gemv_kernel<MR, RPW, KJ, NW, false>), dim3(blocks), dim3(NW * 64), 0, st, a, W, s, c, (int)M, (int)N, (int)K, zp, pt); }
#define HEXMI_GEMV_K(MR) { if (K == 1024) HEXMI_GEMV(MR, 1) else if (K == 2048) HEXMI_GEMV(MR, 2) else if (K == 4096) HEXMI_GEMV(MR, 4) else HEXMI_GEMV(MR, 8) }
    if (M == 1) HEXMI_GEMV_K(1) else HEXMI_GEMV_K(2)
#undef HEXMI_GEMV_K
#undef HEXMI_GEMV
    return launch_status();
  }
  // more than 128 rows with a zero point or a per-tensor scale: the chunked kernel in passes of 128 rows (the tile
  // kernel has no such form; M = 256, N = 11008, K = 4096: 2 x 28 us against four passes of 20 through w8a16_kernel)
  if (((zp || pt) || (K % 64 != 0 && !tile_kernel)) && M > kMidMaxM && K <= (1 << 29)) {
    int rc = HEXMI_OK;
    for (int64_t m = 0; m < M && rc == HEXMI_OK; m += kMidMaxM) {
      const int64_t rows = M - m < kMidMaxM ? M - m : kMidMaxM;
      rc = gemm_w8a16_any(rows, N, K, a + m * K, W, scales, zp, pt, c + m * N, stream);
    }
    return rc;
  }
  // the chunked kernel: any K (a multiple of 16 here)
  if (M <= kMidMaxM && K <= (1 << 29)) {
    const int cus = hexmi_num_cus();
    if (cus <= 0) return HEXMI_ELAUNCH;
    const int64_t per_cu = (N + cus - 1) / cus;
    int chan_per_wg = (int)(per_cu < 16 ? 16 : per_cu);     // one full tile at least
    bool paired = false;
    if (per_cu > kMidCh) {
      // More than a workgroup's 48 channels per CU: equal workgroups in whole rounds over the CUs, not 48 each and
      // a last round of a few (N = 14336, K = 4096, M = 16: 19.3 us that way). Either one workgroup per CU at a
      // time, of up to three channel tiles, or, with up to 16 rows, two of up to two tiles each (their LDS fits
      // twice, so their starts and ends overlap: 14.8 us); whichever copies fewer tile rows, empty ones counted.
      const int64_t r1 = (per_cu + kMidCh - 1) / kMidCh, c1 = (N + cus * r1 - 1) / (cus * r1);
      chan_per_wg = (int)c1;
      if (M <= 16) {
        const int64_t r2 = (per_cu + 63) / 64, c2 = (N + cus * 2 * r2 - 1) / (cus * 2 * r2);
        if (c2 > 16 && r2 * 2 * ((c2 + 15) / 16) <= r1 * ((c1 + 15) / 16)) {
          chan_per_wg = (int)c2;
          paired = true;
        }
      }
    }
    const int64_t grid64 = (N + chan_per_wg - 1) / chan_per_wg;
    if (grid64 > 0x7fffffff) return HEXMI_ENOTSUP;
    const int grid = (int)grid64;
    const int tiles = (chan_per_wg + 15) / 16;              // channel tiles of a workgroup that hold channels
#define HEXMI_MID_T(MB, NT, KC, ZP, TAIL) \
  hipLaunchKernelGGL((w8a16_mid_kernel<MB, NT, KC, ZP, TAIL>), dim3(grid), dim3(1024), 0, st, a, W, s, c, (int)M, (int)N, (int)K, chan_per_wg, paired ? 0 : 1, zp, pt)
  // up to 32 rows the form that takes any K is the only one (its masks and clamps cost nothing there)
#define HEXMI_MID_KC(MB, NT, KC) \
  { if (MB <= 2 || K % KC != 0) { if (zp) HEXMI_MID_T(MB, NT, KC, true, true); else HEXMI_MID_T(MB, NT, KC, false, true); } \
    else { if (zp) HEXMI_MID_T(MB, NT, KC, true, (MB <= 2)); else HEXMI_MID_T(MB, NT, KC, false, (MB <= 2)); } }
#define HEXMI_MID_NT(MB, NT) HEXMI_MID_KC(MB, NT, mid_kc(MB, NT))
#define HEXMI_MID(MB) \
  { if (tiles == 1) HEXMI_MID_NT(MB, 1) else if (tiles == 2) HEXMI_MID_NT(MB, 2) else HEXMI_MID_NT(MB, 3) }
    if (M <= 16) {
      if (paired) HEXMI_MID_KC(1, 2, 256) else HEXMI_MID(1)
    } else if (M <= 32) HEXMI_MID(2) else if (M <= 48) HEXMI_MID(3) else if (M <= 64) HEXMI_MID(4)
    else if (M <= 96) HEXMI_MID(6) else HEXMI_MID(8)
#undef HEXMI_MID
#undef HEXMI_MID_NT
#undef HEXMI_MID_KC
#undef HEXMI_MID_T
    return launch_status();
  }
  if (tile_kernel) return gemm_w8a16_tiled(M, N, K, a, W, s, c, st);
  int rc = HEXMI_OK;
  for (int64_t m = 0; m < M && rc == HEXMI_OK; m += 64) {
    const int64_t left = M - m;
    if (zp || pt) {
      if (left > 32) rc = launch_pass_zp<4>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, zp, pt, st);
      else if (left > 16) rc = launch_pass_zp<2>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, zp, pt, st);
      else rc = launch_pass_zp<1>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, zp, pt, st);
    } else if (left > 32) rc = launch_pass<4>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, st);
    else if (left > 16) rc = launch_pass<2>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, st);
    else rc = launch_pass<1>(a, W, s, c, (int)M, (int)N, (int)K, (int)m, st);
  }
  return rc;
}
}  // namespace

extern "C" int hexmi_gemm_w8a16(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* W, const void* scales,
                                void* C, hexmi_stream_t stream) {
  return gemm_w8a16_any(M, N, K, A, W, scales, nullptr, 0, C, stream);
}

namespace {
// Shapes the (channel range x K part) kernel takes ahead of the kernels of hexmi_gemm_w8a16, from timings of both over
// N in 1024 .. 28672 and K in 2048 .. 14336 on 256 CUs. Those kernels give every workgroup all of K and up to 48
// channels (M <= 128) or a 128 x 128 tile (M > 128): they fall behind when that leaves CUs idle or oversubscribed
// (N > 48 channels per CU, twice that up to 32 rows; fewer tiles than a third of the CUs, or than half of them with
// a long K) and when K is long, since every workgroup pulls M x K of activations through L2: up to 96 rows from
// K = 8192 on and only when K is more than twice N (N = 4096, K = 8192, M = 64: 23.4 us against 26.0; K = 11008:
// 29.4 against 28.9), above 96 rows from K = 4608 + 64 per channel of a CU's share on (N = 4096: 27.6 against 28.6 us
// at K = 5120, 31.7 against 29.7 at 6144; N = 11008: 41.4 against 42.5 at K = 7168, 47.6 against 44.6 at 8192).
bool prefer_split(int64_t M, int64_t N, int64_t K, int cus) {
  if (M < 32 || M > 256) return false;
  if (M <= 32) return N > 96 * (int64_t)cus;
  if (M <= 128) {
    if (N > 48 * (int64_t)cus) return true;
    if (M <= 96) return K >= 8192 && K > 2 * N;
    return K >= 4608 + 64 * ((N + cus - 1) / cus);
  }
  const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
  return tiles * 3 <= cus || (tiles * 2 <= cus && K >= 8192);
}
}  // namespace

extern "C" int64_t hexmi_gemm_w8a16_workspace(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int cus = hexmi_num_cus();
  if (cus <= 0 || !prefer_split(M, N, K, cus)) return 0;
  return w8a16_split_workspace(M, N, K, cus);
}

extern "C" int hexmi_gemm_w8a16_ws(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* W, const void* scales,
                                   void* C, void* workspace, int64_t workspace_bytes, hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0 || workspace_bytes < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!C || (K > 0 && (!A || !W || !scales))) return HEXMI_EINVAL;
  const int cus = hexmi_num_cus();
  if (cus > 0 && K > 0 && prefer_split(M, N, K, cus) && (workspace || w8a16_split_workspace(M, N, K, cus) == 0)) {
    const int64_t need = w8a16_split_workspace(M, N, K, cus);
    if (need > 0 && workspace_bytes < need) return HEXMI_EINVAL;
    hipStream_t st = as_stream(stream);
    begin_call();
    int rc = HEXMI_OK;
    if (need > 0) {
      // the flags the K parts raise start at zero in every call: the workspace carries nothing from one call to the next
      rc = w8a16_split_clear(workspace, w8a16_split_header(M, N, K, cus), st);
      if (rc != HEXMI_OK) return rc;
    }
    if (w8a16_split(M, N, K, static_cast<const f16*>(A), W, static_cast<const f16*>(scales), static_cast<f16*>(C),
                    workspace, workspace_bytes, cus, st, &rc))
      return rc;
  }
  return hexmi_gemm_w8a16(M, N, K, A, W, scales, C, stream);
}

extern "C" int hexmi_pack_w8(int64_t N, int64_t K, const int8_t* W, int8_t* Wp, hexmi_stream_t stream) {
  if (N < 0 || K < 0) return HEXMI_EINVAL;
  if (N == 0 || K == 0) return HEXMI_OK;
  if (!W || !Wp) return HEXMI_EINVAL;
  if (K % 64 != 0) return HEXMI_ENOTSUP;
  if (!aligned_to(W, 16) || !aligned_to(Wp, 16)) return HEXMI_EINVAL;
  const int64_t chunks = ((N + 15) / 16) * 16 * (K / 16);   // 16-byte chunks of the packed buffer
  const int64_t blocks = (chunks + 255) / 256;
  if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
  begin_call();
  hipLaunchKernelGGL(pack_w8_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), W, Wp, N, K, chunks);
  return launch_status();
}

extern "C" int hexmi_gemm_w8a16_packed(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* Wp,
                                       const void* scales, void* C, hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!A || !Wp || !scales || !C) return HEXMI_EINVAL;
  // the K slices of the 16 waves are whole 64-wide steps, at most four each
  if (K == 0 || K % (kPWaves * 64) != 0 || K / (kPWaves * 64) > kPSteps) return HEXMI_ENOTSUP;
  if (!aligned_to(A, 16) || !aligned_to(Wp, 16)) return HEXMI_EINVAL;
  if (M > 0x7fffffff || N > 0x7fffffff - 16) return HEXMI_ENOTSUP;
  const int cus = hexmi_num_cus();
  if (cus <= 0) return HEXMI_ELAUNCH;
  hipStream_t st = as_stream(stream);
  begin_call();
  const int64_t tiles = (N + 15) / 16;
  const int tiles_per_wg = (int)((tiles + cus - 1) / cus);
  const int chan_per_wg = tiles_per_wg * 16;
  const int grid = (int)((tiles + tiles_per_wg - 1) / tiles_per_wg);
  // sixteen activation rows per launch: more rows walk the packed weights again (they then come from the caches)
  int rc = HEXMI_OK;
  for (int64_t m = 0; m < M && rc == HEXMI_OK; m += 16) {
    const int rows = (int)(M - m < 16 ? M - m : 16);
    hipLaunchKernelGGL(w8a16_persist_kernel, dim3(grid), dim3(1024), 0, st, static_cast<const f16*>(A) + m * K, Wp,
                       static_cast<const f16*>(scales), static_cast<f16*>(C) + m * N, rows, (int)N, (int)K, chan_per_wg);
    rc = launch_status();
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
  begin_call();
  hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), W,
                     static_cast<const f16*>(scales), out, N, K);
  return launch_status();
}

// ---- quant.dcast with a zero point and / or per-tensor parameters ------------------------------------------------

extern "C" int hexmi_dequant_w8_ex(int64_t N, int64_t K, const int8_t* W, const void* scales, const int8_t* zero_points,
                                   int per_tensor, float* out, hexmi_stream_t stream) {
  if (N < 0 || K < 0) return HEXMI_EINVAL;
  if (N == 0 || K == 0) return HEXMI_OK;
  if (!W || !scales || !out) return HEXMI_EINVAL;
  const int64_t total = N * K;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  begin_call();
  hipLaunchKernelGGL(dequant_ex_kernel, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), W,
                     static_cast<const f16*>(scales), zero_points, per_tensor ? 1 : 0, out, N, K);
  return launch_status();
}

extern "C" int hexmi_gemm_w8a16_ex(int64_t M, int64_t N, int64_t K, const void* A, const int8_t* W, const void* scales,
                                   const int8_t* zero_points, int per_tensor, void* C, hexmi_stream_t stream) {
  return gemm_w8a16_any(M, N, K, A, W, scales, zero_points, per_tensor ? 1 : 0, C, stream);
}
