// Dense GEMM C[M,N] = A[M,K] * op(B) on gfx950 matrix cores (fp16 / bf16 in, fp32 accumulate).
//
// Workgroup = 256 threads = 4 waves in a 2x2 arrangement; each wave owns a (WM*32) x (WN*32) block of C as
// WM x WN accumulators of v_mfma_f32_32x32x16 (4x4 = 256 accumulator registers for the 256x256 tile). The K loop
// walks 32-wide slabs through FOUR LDS stages. A slab of A (and of B) is copied global -> LDS by
// global_load_lds_dwordx4 (no register staging); the copy of slab kt+3 is issued while slab kt is multiplied,
// spread between the MFMAs, and one s_barrier per slab both publishes slab kt+1 and frees the stage of slab kt-1.
// Fragments are double buffered in registers across that barrier: the LDS reads of the next 16-wide k step are
// issued between the MFMAs of the current one (sched_group_barrier pins the interleaving). Each stage of each
// operand is its own LDS object so the compiler's wait-count tracking keeps reads of one stage independent of
// copies into another.
//
// LDS layouts (16-byte chunks, XOR swizzled through the *source* address each lane fetches, since the LDS side
// of a global_load_lds is fixed at base + lane*16):
//   K-contiguous operand (A, and B given as [N,K]): [row][4 chunks]; chunk c of row r sits at c ^ ((r>>2)&3).
//     A fragment is one ds_read_b128 per lane (row = lane%32, 8 consecutive k).
//   N-contiguous operand (B given as [K,N]): [k][BN/8 chunks]; chunk c of row k sits at c ^ ((k&3)<<2).
//     A fragment is two ds_read_b64_tr_b16: the transposing LDS read hands each lane 4 consecutive k of one column.
//
// The MFMA is issued with the B fragment as its first operand, so a lane's 4 consecutive accumulator registers
// are 4 consecutive columns of one C row and go out as one 8-byte (fp16/bf16) or 16-byte (fp32) store.
//
// Which kernel takes a product (dispatch_gemm): operand rows on 16-byte boundaries and whole 64-wide (gemm_kernel_k64)
// or 32-wide (gemm_kernel) slabs of K -> the tiled kernels as described; K a multiple of 8 only -> gemm_kernel with
// the last slab's chunks past K fetched from a zero chunk; an output side without runs of four columns (odd N with B
// as [N,K], odd ldc, unaligned C) -> the same kernels with the tile leaving through LDS one element per lane;
// anything else (unaligned operand rows, K % 8 != 0) -> gemm_kernel_any, which stages the slabs through registers.
// Up to eight rows against B as [N,K] -> gemv_nt_kernel, a stream of the weights with one wave per output channel.
// Nine to 64 rows against B as [N,K], where a fitted cost says so -> gemm_nt_skinny_kernel, a workgroup per 16 channels.
#include <algorithm>
#include <type_traits>

#include "hexmi_common.h"

namespace hexmi {
namespace {

#define HEXMI_LDS(p) ((__attribute__((address_space(3))) void*)(p))
#define HEXMI_GLB(p) ((const __attribute__((address_space(1))) void*)(p))

constexpr int BK = 32;                 // K extent of a slab (elements)
constexpr int kChunk = 8;              // elements per 16-byte chunk

template <typename T> struct Mfma;
template <> struct Mfma<f16> {
  typedef f16x8 Frag;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<bf16> {
  typedef bf16x8 Frag;
  static __device__ __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

// Sixteen zero bytes in device memory: where a copy lane of the ragged-K kernel points when its chunk lies past K.
__device__ __attribute__((aligned(16))) unsigned g_zero_chunk[4];

__device__ __forceinline__ int swz_k(int row) { return (row >> 2) & 3; }      // K-contiguous tiles
__device__ __forceinline__ int swz_n(int k) { return (k & 3) << 2; }          // N-contiguous tiles

// s_waitcnt immediate (gfx9 encoding): at most `vm` vector-memory operations outstanding, all LDS reads returned.
constexpr int waitcnt_imm(int vm) { return (vm & 0xF) | ((vm >> 4) << 14) | (7 << 4) | (0 << 8); }

// global -> LDS copy of a [ROWS x 32] K-contiguous slab: ROWS/64 wave-wide instructions per wave, 16 rows each.
// Rows past row_max are clamped (their products are never stored).
template <typename T, int ROWS, int NW = 4>
struct KMajorLoader {
  static constexpr int NI = ROWS / (16 * NW);
  const T* ptr[NI];
  int lds_off[NI];
  int kc[NI];                                       // first k of this lane's chunk within the slab
  __device__ __forceinline__ void init(const T* g, int64_t ld, int row0, int row_max, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * NW + wave;
      const int row = inst * 16 + lane / 4;
      const int c = (lane % 4) ^ swz_k(row);
      int grow = row0 + row;
      grow = grow < row_max ? grow : row_max;
      ptr[j] = g + (int64_t)grow * ld + c * kChunk;
      lds_off[j] = inst * 16 * BK;
      kc[j] = c * kChunk;
    }
  }
  template <int J> __device__ __forceinline__ void issue(T* lds, int k0) const {
    __builtin_amdgcn_global_load_lds(HEXMI_GLB(ptr[J] + k0), HEXMI_LDS(lds + lds_off[J]), 16, 0, 0);
  }
  // K % 8 == 0 but not a whole number of slabs: a chunk starting at or past K is fetched from the zero chunk
  template <int J> __device__ __forceinline__ void issue_ragged(T* lds, int k0, int K) const {
    const T* src = k0 + kc[J] < K ? ptr[J] + k0 : reinterpret_cast<const T*>(g_zero_chunk);
    __builtin_amdgcn_global_load_lds(HEXMI_GLB(src), HEXMI_LDS(lds + lds_off[J]), 16, 0, 0);
  }
};

// global -> LDS copy of a [32 x COLS] N-contiguous slab; column chunks past col_max are clamped.
template <typename T, int COLS, int NW = 4>
struct NMajorLoader {
  static constexpr int NI = COLS / (16 * NW);
  static constexpr int CPR = COLS / kChunk;         // chunks per row
  const T* ptr[NI];
  int lds_off[NI];
  int krow[NI];                                     // row of the slab this lane's chunk belongs to
  int64_t ld;
  __device__ __forceinline__ void init(const T* g, int64_t ld_, int col0, int col_max, int wave, int lane) {
    ld = ld_;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * NW + wave;
      const int lin = inst * 64 + lane;
      const int k = lin / CPR;
      const int c = (lin % CPR) ^ swz_n(k);
      int gcol = col0 + c * kChunk;
      gcol = gcol < col_max ? gcol : col_max;
      ptr[j] = g + (int64_t)k * ld + gcol;
      lds_off[j] = inst * 64 * kChunk;
      krow[j] = k;
    }
  }
  template <int J> __device__ __forceinline__ void issue(T* lds, int k0) const {
    __builtin_amdgcn_global_load_lds(HEXMI_GLB(ptr[J] + (int64_t)k0 * ld), HEXMI_LDS(lds + lds_off[J]), 16, 0, 0);
  }
  // a slab that reaches past K: the rows at or past K are fetched from the zero chunk
  template <int J> __device__ __forceinline__ void issue_ragged(T* lds, int k0, int K) const {
    const T* src = k0 + krow[J] < K ? ptr[J] + (int64_t)k0 * ld : reinterpret_cast<const T*>(g_zero_chunk);
    __builtin_amdgcn_global_load_lds(HEXMI_GLB(src), HEXMI_LDS(lds + lds_off[J]), 16, 0, 0);
  }
};

// Weight-only quantised B: a [ROWS x 32] int8 K-contiguous slab is copied global -> LDS raw (16-byte chunk
// (row, half) at linear position row*2 + half, no swizzle), and one slab later converted LDS -> LDS into the same
// swizzled fp16 K-contiguous tile a global_load_lds copy of fp16 data would have filled. All global traffic stays
// on the asynchronous copy path, so one in-order counter paces A and B alike.
template <int ROWS>
struct I8Loader {
  static constexpr int NI = ROWS / 128 > 0 ? ROWS / 128 : 1;   // copy instructions per wave per slab
  static constexpr int NC = ROWS * 2 / 256;                    // 16-byte chunks converted per thread per slab
  const int8_t* ptr[NI];
  int raw_off[NI];
  int cv_raw[NC];                                             // raw byte offset of this thread's chunk
  int cv_el[NC][2];                                           // fp16 element offsets of the two chunks it expands to
  __device__ __forceinline__ void init(const int8_t* g, int64_t ld, int row0, int row_max, int wave, int lane,
                                       int tid) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * 4 + wave;
      const int idx = inst * 64 + lane;
      const int row = idx / 2, half = idx % 2;
      int grow = row0 + row;
      grow = grow < row_max ? grow : row_max;
      ptr[j] = g + (int64_t)grow * ld + half * 16;
      raw_off[j] = inst * 64 * 16;
    }
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const int idx = j * 256 + tid;
      const int row = idx / 2, half = idx % 2;
      cv_raw[j] = idx * 16;
      cv_el[j][0] = row * BK + (((half * 2 + 0) ^ swz_k(row)) * kChunk);
      cv_el[j][1] = row * BK + (((half * 2 + 1) ^ swz_k(row)) * kChunk);
    }
  }
  template <int J> __device__ __forceinline__ void issue(int8_t* raw, int k0) const {
    if constexpr (J < NI)
      __builtin_amdgcn_global_load_lds(HEXMI_GLB(ptr[J] + k0), HEXMI_LDS(raw + raw_off[J]), 16, 0, 0);
  }
  __device__ __forceinline__ void convert(const int8_t* raw, f16* lds) const {
#pragma unroll
    for (int j = 0; j < NC; ++j) {
      const u32x4 r = *reinterpret_cast<const u32x4*>(raw + cv_raw[j]);
      f16x8 w0, w1;
      cvt16(r, w0, w1);
      *reinterpret_cast<f16x8*>(lds + cv_el[j][0]) = w0;
      *reinterpret_cast<f16x8*>(lds + cv_el[j][1]) = w1;
    }
  }
};

template <typename T>
__device__ __forceinline__ typename Mfma<T>::Frag read_kmajor(const T* lds, int row, int chunk) {
  typedef typename Mfma<T>::Frag Frag;
  return *reinterpret_cast<const Frag*>(lds + row * BK + ((chunk ^ swz_k(row)) * kChunk));
}

template <typename T, int COLS>
__device__ __forceinline__ typename Mfma<T>::Frag read_nmajor(const T* lds, int col_tile, int ks, int lane) {
  typedef typename Mfma<T>::Frag Frag;
  constexpr int CPR = COLS / kChunk;
  const int g = lane / 16, i = lane % 16;
  const int n = col_tile + (g & 1) * 16 + (i & 3) * 4;    // 4 consecutive columns fetched by this lane
  const int kb = ks * 16 + (g >> 1) * 8 + (i >> 2);
  union { i16x4 h[2]; Frag f; } u;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int k = kb + p * 4;
    const int c = (n / kChunk) ^ swz_n(k);
    const T* addr = lds + (k * CPR + c) * kChunk + (n % kChunk);
    u.h[p] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(addr));
  }
  return u.f;
}

// Map the linear workgroup id to a C tile: consecutive ids go to different XCDs (each with its own L2), so
// first give every XCD a contiguous run of logical ids, then walk tiles in bands of GROUP_M tile-rows so the
// tiles resident on one XCD share A and B panels.
__device__ __forceinline__ void tile_of_block(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  // XCD x runs ids x, x + 8, ...: total/8 of them, one more on the first total%8 XCDs
  const int xcd = pid % 8, per = total / 8, extra = total % 8;
  const int logical = xcd * per + (xcd < extra ? xcd : extra) + pid / 8;
  constexpr int GROUP_M = 4;
  const int group_size = GROUP_M * tiles_n;
  const int group = logical / group_size;
  const int first_m = group * GROUP_M;
  const int gm = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
  const int in_group = logical % group_size;
  tm = first_m + in_group % gm;
  tn = in_group / gm;
}

// Epilogue operands of hexmi_gemm_ex: C = A B + bias[column] + residual[row, column], both of the output type, added
// to the fp32 sums before the one rounding to the output type. ok4: the four columns col .. col+3 exist and the
// operands may be read as one 4-element run (the fast kernels: N % 8 == 0, ldr % 4 == 0, aligned bases).
// The output pointer of a tiled kernel: declared without aliasing (as every operand pointer here is) except in the
// instantiations that add a residual, which may be the output buffer itself.
template <typename P, bool MAY_ALIAS> struct OutPtr { typedef P* __restrict__ type; };
template <typename P> struct OutPtr<P, true> { typedef P* type; };

template <typename OutT> struct Run4;
template <> struct Run4<float> { typedef f32x4 V; };
template <> struct Run4<f16> { typedef f16x4 V; };
template <> struct Run4<bf16> { typedef bf16x4 V; };
template <typename OutT>
__device__ __forceinline__ void add_epilogue4(f32x4& a, const OutT* __restrict__ bias, const OutT* resid,
                                              int64_t ldr, int row, int col) {
  typedef typename Run4<OutT>::V V;
  if (bias) {
    const V b = *reinterpret_cast<const V*>(bias + col);
#pragma unroll
    for (int r = 0; r < 4; ++r) a[r] += to_f32<OutT>(b[r]);
  }
  if (resid) {
    const V v = *reinterpret_cast<const V*>(resid + (int64_t)row * ldr + col);
#pragma unroll
    for (int r = 0; r < 4; ++r) a[r] += to_f32<OutT>(v[r]);
  }
}

// The output tile of a workgroup (waves 2 x NWN, each WM x WN MFMA tiles of 32x32) leaves through LDS in rows, for
// output sides that allow no runs of four columns (an odd N or leading dimension, an unaligned base). Storing a
// lane's accumulators one by one would be 64 pieces of 64 different rows per instruction (measured: 876 us against
// 324 for the aligned neighbour of [4096, 768] x [50257, 768]^T), so the tile is staged kRows rows at a time -- a
// pass takes its rows of one MFMA tile row from the waves that hold it -- and leaves in the aligned 16-byte pieces
// of each row. Bias and residual are added on the way in, element by element (a residual
// that is the output buffer is read before any element of the pass is stored).
// c_s: kRows x (BN + 4) elements: 32 rows of 16-bit results or 16 of fp32 (8.25 KiB at BN = 128); the pitch keeps the
// rows of a wave's 8- or 16-byte writes on different banks.
template <typename OutT> struct RaggedStage {
  static constexpr int kRows = sizeof(OutT) == 4 ? 16 : 32;
  static constexpr int pitch(int bn) { return bn + 4; }
};
template <typename OutT, int WM, int WN, int NW, int BM, int BN>
__device__ __forceinline__ void store_tile_by_rows(const f32x16 (&acc)[WM][WN], OutT* c_s, OutT* C, int64_t ldc,
                                                   const OutT* bias, const OutT* resid, int64_t ldr, int M, int N, int m0,
                                                   int n0, int wm, int wn, int wave, int lane,
                                                   const f16* scales = nullptr, int per_tensor = 0) {
  constexpr int PR = RaggedStage<OutT>::kRows, PITCH = RaggedStage<OutT>::pitch(BN);
#pragma unroll
  for (int p = 0; p < BM / PR; ++p) {
    const int t = p * PR / 32, sub = p * PR % 32;          // MFMA tile row of the workgroup tile; first row inside it
    const int lr32 = lane % 32;
    if (wm == t / WM && lr32 >= sub && lr32 < sub + PR) {
      const int row = m0 + t * 32 + lr32;
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = (wn * WN + j) * 32 + 8 * q + 4 * (lane / 32);
          f32x4 c = {acc[t % WM][j][q * 4 + 0], acc[t % WM][j][q * 4 + 1], acc[t % WM][j][q * 4 + 2],
                     acc[t % WM][j][q * 4 + 3]};
          if (scales) {                                  // weight-only quantised B: the channel scale on the finished sum
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (n0 + col + r < N) c[r] *= (float)scales[per_tensor ? 0 : n0 + col + r];
          }
          if (bias || resid) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (row < M && n0 + col + r < N) {
                if (bias) c[r] += to_f32<OutT>(bias[n0 + col + r]);
                if (resid) c[r] += to_f32<OutT>(resid[(int64_t)row * ldr + n0 + col + r]);
              }
          }
          store4<OutT>(&c_s[(lr32 - sub) * PITCH + col], c[0], c[1], c[2], c[3]);
        }
    }
    __syncthreads();
    // the staged rows leave in the aligned 16-byte pieces each holds (a lane gathers a piece's elements), the up to
    // E - 1 elements before a row's first boundary and after its last whole piece by elements, a lane per row
    constexpr int E = 16 / (int)sizeof(OutT), CPR = BN / E;
    const int ncols = N - n0 < BN ? N - n0 : BN;
    const int64_t c_elem = (int64_t)(reinterpret_cast<uintptr_t>(C) / sizeof(OutT));
    auto lead_of = [&](int64_t e0) { return (int)((E - ((c_elem + e0) & (E - 1))) & (E - 1)); };
    const int tid = wave * 64 + lane;
#pragma unroll
    for (int idx = tid; idx < PR * CPR; idx += NW * 64) {
      const int lr = idx / CPR, q = idx % CPR, row = m0 + p * PR + lr;
      const int64_t e0 = (int64_t)row * ldc + n0;
      const int c0 = lead_of(e0) + E * q;
      if (row < M && c0 + E <= ncols) {
        __attribute__((aligned(16))) OutT o[E];
#pragma unroll
        for (int i = 0; i < E; ++i) o[i] = c_s[lr * PITCH + c0 + i];
        *reinterpret_cast<u32x4*>(C + e0 + c0) = *reinterpret_cast<const u32x4*>(o);
      }
    }
    // (every read of the staged row ahead of the first store, the stores under masks: a loop with one read and one
    // store per turn would put a pass's worth of LDS latencies end to end on one wave while the others wait)
    if (tid < 2 * PR && m0 + p * PR + tid % PR < M && ncols > 0) {
      const int lr = tid % PR;
      const int64_t e0 = (int64_t)(m0 + p * PR + lr) * ldc + n0;
      const int lead = lead_of(e0);
      // lanes 0 .. PR - 1: the columns before the first boundary; PR .. 2 PR - 1: those after the last whole piece
      const int from = tid < PR ? 0 : (ncols > lead ? lead + ((ncols - lead) & ~(E - 1)) : ncols);
      const int to = tid < PR ? (lead < ncols ? lead : ncols) : ncols;
      OutT ends[E - 1];
#pragma unroll
      for (int k = 0; k < E - 1; ++k) ends[k] = c_s[lr * PITCH + (from + k < BN ? from + k : BN - 1)];
#pragma unroll
      for (int k = 0; k < E - 1; ++k)
        if (from + k < to) C[e0 + from + k] = ends[k];
    }
    __syncthreads();
  }
}

// K % 32 == 0. TAIL: the slab count is not a multiple of 4, so the last pass over the four stages guards its MFMAs.
// B_I8: B is int8 [N,K] (weight-only quantisation, needs TRANS_B and T = fp16); its slabs are copied raw into
// LDS, converted to fp16 LDS -> LDS one slab later, and the result is multiplied by scales[column].
// NWN: waves along N (2: four waves, one per SIMD, each WM x WN tiles of 32x32; 4: eight waves, two per SIMD).
// The eight-wave 256x256 form (WM = 4, WN = 2) measured the same as four waves with 4x4 tiles on both benchmark
// shapes: on random data the kernel is held back by the power limit, not by issue stalls a second wave could fill.
// RAGGED (with TAIL and EPI): K is a multiple of 8 only -- the last slab's chunks past K come from a zero chunk --
// and the output side may be anything: with run_epilogue == 0 (N, the leading dimensions of C and the residual or a
// base address do not allow runs of four columns) bias, residual and C are touched one element at a time.
template <typename T, typename OutT, int WM, int WN, bool TRANS_B, bool TAIL, bool B_I8 = false, int NWN = 2,
          bool EPI = false, bool RAGGED = false>
__global__ __launch_bounds__(NWN * 128)
void gemm_kernel(const T* __restrict__ A, const void* __restrict__ Bv, typename OutPtr<OutT, EPI>::type C, int M, int N, int K,
                 int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n,
                 const f16* __restrict__ scales = nullptr, const OutT* __restrict__ bias = nullptr,
                 const OutT* resid = nullptr, int64_t ldr = 0, int run_epilogue = 1) {
  static_assert(!RAGGED || (TAIL && EPI && !B_I8), "the ragged form carries the guarded last pass and the epilogue operands");
  const T* B = static_cast<const T*>(Bv);
  typedef typename Mfma<T>::Frag Frag;
  constexpr int NW = 2 * NWN;                       // waves per workgroup
  constexpr int BM = 2 * WM * 32, BN = NWN * WN * 32;
  static_assert(!B_I8 || NWN == 2, "the int8 loader is written for four waves");
  __shared__ __attribute__((aligned(16))) T a_s0[BM * BK];
  __shared__ __attribute__((aligned(16))) T a_s1[BM * BK];
  __shared__ __attribute__((aligned(16))) T a_s2[BM * BK];
  __shared__ __attribute__((aligned(16))) T a_s3[BM * BK];
  __shared__ __attribute__((aligned(16))) T b_s0[BN * BK];
  __shared__ __attribute__((aligned(16))) T b_s1[BN * BK];
  __shared__ __attribute__((aligned(16))) T b_s2[BN * BK];
  __shared__ __attribute__((aligned(16))) T b_s3[BN * BK];
  // raw int8 B slabs on their way to fp16 (weight-only quantised B only)
  __shared__ __attribute__((aligned(16))) int8_t r_s0[B_I8 ? BN * BK : 16];
  __shared__ __attribute__((aligned(16))) int8_t r_s1[B_I8 ? BN * BK : 16];
  __shared__ __attribute__((aligned(16))) int8_t r_s2[B_I8 ? BN * BK : 16];
  __shared__ __attribute__((aligned(16))) int8_t r_s3[B_I8 ? BN * BK : 16];
  // rows of the output tile on their way out (ragged output side only; two workgroups still fit a CU)
  __shared__ __attribute__((aligned(16))) OutT c_s[RAGGED ? RaggedStage<OutT>::kRows * RaggedStage<OutT>::pitch(BN) : 8];

  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int wm = wave / NWN, wn = wave % NWN;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  KMajorLoader<T, BM, NW> load_a;
  load_a.init(A, lda, m0, M - 1, wave, lane);
  KMajorLoader<T, BN, NW> load_bk;
  NMajorLoader<T, BN, NW> load_bn;
  I8Loader<BN> load_b8;
  if constexpr (B_I8) load_b8.init(static_cast<const int8_t*>(Bv), ldb, n0, N - 1, wave, lane, threadIdx.x);
  else if constexpr (TRANS_B) load_bk.init(B, ldb, n0, N - 1, wave, lane);
  else load_bn.init(B, ldb, n0, N - kChunk, wave, lane);
  constexpr int NLA = BM / (16 * NW);               // copy instructions per wave per slab (A)
  constexpr int NLB = B_I8 ? I8Loader<BN>::NI : BN / (16 * NW);   // B copies per wave per slab

  // part 0 = the A copies of slab kt, part 1 = its B copies
  auto issue_part = [&](int kt, T* a_dst, T* b_dst, auto part) {
    constexpr int P = decltype(part)::value;
    const int k0 = kt * BK;
    if constexpr (RAGGED) {
      if constexpr (P == 0) {
        load_a.template issue_ragged<0>(a_dst, k0, K);
        if constexpr (NLA > 1) load_a.template issue_ragged<1>(a_dst, k0, K);
        if constexpr (NLA > 2) load_a.template issue_ragged<2>(a_dst, k0, K);
        if constexpr (NLA > 3) load_a.template issue_ragged<3>(a_dst, k0, K);
      } else if constexpr (TRANS_B) {
        load_bk.template issue_ragged<0>(b_dst, k0, K);
        if constexpr (NLB > 1) load_bk.template issue_ragged<1>(b_dst, k0, K);
        if constexpr (NLB > 2) load_bk.template issue_ragged<2>(b_dst, k0, K);
        if constexpr (NLB > 3) load_bk.template issue_ragged<3>(b_dst, k0, K);
      } else {
        load_bn.template issue_ragged<0>(b_dst, k0, K);
        if constexpr (NLB > 1) load_bn.template issue_ragged<1>(b_dst, k0, K);
        if constexpr (NLB > 2) load_bn.template issue_ragged<2>(b_dst, k0, K);
        if constexpr (NLB > 3) load_bn.template issue_ragged<3>(b_dst, k0, K);
      }
    } else if constexpr (P == 0) {
      load_a.template issue<0>(a_dst, k0);
      if constexpr (NLA > 1) load_a.template issue<1>(a_dst, k0);
      if constexpr (NLA > 2) load_a.template issue<2>(a_dst, k0);
      if constexpr (NLA > 3) load_a.template issue<3>(a_dst, k0);
    } else if constexpr (B_I8) {
      // nothing: int8 B goes through registers (see the slab body)
    } else if constexpr (TRANS_B) {
      load_bk.template issue<0>(b_dst, k0);
      if constexpr (NLB > 1) load_bk.template issue<1>(b_dst, k0);
      if constexpr (NLB > 2) load_bk.template issue<2>(b_dst, k0);
      if constexpr (NLB > 3) load_bk.template issue<3>(b_dst, k0);
    } else {
      load_bn.template issue<0>(b_dst, k0);
      if constexpr (NLB > 1) load_bn.template issue<1>(b_dst, k0);
      if constexpr (NLB > 2) load_bn.template issue<2>(b_dst, k0);
      if constexpr (NLB > 3) load_bn.template issue<3>(b_dst, k0);
    }
  };
  auto read_frags = [&](const T* a_src, const T* b_src, int ks, Frag* af, Frag* bf) {
#pragma unroll
    for (int i = 0; i < WM; ++i) af[i] = read_kmajor<T>(a_src, (wm * WM + i) * 32 + lane % 32, ks * 2 + lane / 32);
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      if constexpr (TRANS_B || B_I8) bf[j] = read_kmajor<T>(b_src, (wn * WN + j) * 32 + lane % 32, ks * 2 + lane / 32);
      else bf[j] = read_nmajor<T, BN>(b_src, (wn * WN + j) * 32, ks, lane);
    }
  };
  auto mfma_all = [&](const Frag* af, const Frag* bf) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[i][j] = Mfma<T>::run(bf[j], af[i], acc[i][j]);
  };
  // Pin the issue order of one group (NREAD LDS reads, NV copies, NMFMA MFMAs) in four identical rounds.
  constexpr int NREAD = WM + ((TRANS_B || B_I8) ? WN : 2 * WN);
  constexpr int NMFMA = WM * WN;
  auto interleave = [&](auto nvmem) {
    constexpr int NV = decltype(nvmem)::value;
    if constexpr (NMFMA >= 8) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                       // LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                       // MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, (NV + 3) / 4, 0);            // VMEM read (the copies)
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (NREAD + 3) / 4 - 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, NMFMA / 4 - 2, 0);
      }
    }
  };
  constexpr int L = NLA + NLB;
  const int KT = RAGGED ? (K + BK - 1) / BK : K / BK;
  auto clampk = [&](int kt) { return kt < KT ? kt : KT - 1; };   // past the end: reload the last slab (never used)
  std::integral_constant<int, 0> part_a;
  std::integral_constant<int, 1> part_b;
  std::integral_constant<int, NLA> n_a;
  std::integral_constant<int, NLB> n_b;

  Frag af[2][WM], bf[2][WN];
  auto issue_raw = [&](int kt, int8_t* raw) {
    load_b8.template issue<0>(raw, kt * BK);
    load_b8.template issue<1>(raw, kt * BK);
  };
  issue_part(0, a_s0, b_s0, part_a);
  issue_part(0, a_s0, b_s0, part_b);
  issue_part(clampk(1), a_s1, b_s1, part_a);
  issue_part(clampk(1), a_s1, b_s1, part_b);
  issue_part(clampk(2), a_s2, b_s2, part_a);
  issue_part(clampk(2), a_s2, b_s2, part_b);
  if constexpr (B_I8) {
    // raw slabs 0..2 are in flight; 0 and 1 are converted before the loop, 2 by the first slab body
    issue_raw(0, r_s0);
    issue_raw(clampk(1), r_s1);
    issue_raw(clampk(2), r_s2);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(NLB));            // A 0..2 and raw 0, 1 landed
    __builtin_amdgcn_s_barrier();
    load_b8.convert(r_s0, reinterpret_cast<f16*>(b_s0));
    load_b8.convert(r_s1, reinterpret_cast<f16*>(b_s1));
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(B_I8 ? NLB : 2 * L));   // slab 0 landed (and the conversions written)
  __builtin_amdgcn_s_barrier();
  read_frags(a_s0, b_s0, 0, af[0], bf[0]);

  // One slab. Slab kt lives in stage kt%4 = (ac, bc); (an, bn) is the stage of slab kt+1; (afree, bfree) is the
  // stage of slab kt-1, released by the barrier that preceded this body, and receives slab kt+3.
  // At the barrier in the middle the copies still allowed in flight are slab kt+2 and the A part of slab kt+3,
  // so slab kt+1 has landed for every wave that passes it; every wave has also issued (and, by the lgkmcnt(0)
  // in the same wait, completed) its last LDS read of slab kt, which frees stage kt%4 for the next body.
  // int8 B: the raw copy of slab kt+3 goes to rfree with the A copies; the barrier in the middle then only lets
  // this body's own copies stay in flight, so raw slab kt+2 (r2) has landed and is converted into its fp16 stage
  // b2 in the second half -- a stage freed two barriers ago and first read after the next body's barrier.
#define HEXMI_SLAB(ac, bc, an, bn, afree, bfree, rfree, r2, b2, kt)   \
  {                                                                   \
    issue_part(clampk((kt) + 3), afree, bfree, part_a);               \
    if constexpr (B_I8) issue_raw(clampk((kt) + 3), rfree);           \
    read_frags(ac, bc, 1, af[1], bf[1]);                              \
    if (!TAIL || (kt) < KT) mfma_all(af[0], bf[0]);                   \
    interleave(n_a);                                                  \
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(B_I8 ? NLA + NLB : L + NLA));   \
    __builtin_amdgcn_s_barrier();                                     \
    issue_part(clampk((kt) + 3), afree, bfree, part_b);               \
    if constexpr (B_I8) load_b8.convert(r2, reinterpret_cast<f16*>(b2));   \
    read_frags(an, bn, 0, af[0], bf[0]);                              \
    if (!TAIL || (kt) < KT) mfma_all(af[1], bf[1]);                   \
    interleave(n_b);                                                  \
  }
  for (int kt = 0; kt < KT; kt += 4) {
    HEXMI_SLAB(a_s0, b_s0, a_s1, b_s1, a_s3, b_s3, r_s3, r_s2, b_s2, kt);
    HEXMI_SLAB(a_s1, b_s1, a_s2, b_s2, a_s0, b_s0, r_s0, r_s3, b_s3, kt + 1);
    HEXMI_SLAB(a_s2, b_s2, a_s3, b_s3, a_s1, b_s1, r_s1, r_s0, b_s0, kt + 2);
    HEXMI_SLAB(a_s3, b_s3, a_s0, b_s0, a_s2, b_s2, r_s2, r_s1, b_s1, kt + 3);
  }
#undef HEXMI_SLAB
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));       // drain the trailing copies before the workgroup's LDS goes away

  // acc[i][j][r]: row = lane%32 of the 32x32 tile, column = 8*(r/4) + 4*(lane/32) + r%4.
  if constexpr (RAGGED) {
    if (!run_epilogue) {
      store_tile_by_rows<OutT, WM, WN, NW, BM, BN>(acc, c_s, C, ldc, bias, resid, ldr, M, N, m0, n0, wm, wn, wave, lane);
      return;
    }
  }
  if constexpr (EPI) {
    // bias and residual join the fp32 sums in registers, all loads issued before the first store (so the residual
    // may be the output buffer itself)
    static_assert(!B_I8, "the epilogue operands go with fp16 / bf16 B");
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      int row = m0 + (wm * WM + i) * 32 + lane % 32;
      row = row < M ? row : M - 1;                  // past the edge: any valid row, those rows are not stored
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          int col = n0 + (wn * WN + j) * 32 + 8 * q + 4 * (lane / 32);
          col = col < N - 4 ? col : N - 4;
          f32x4 c = {acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
          add_epilogue4<OutT>(c, bias, resid, ldr, row, col);
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][j][q * 4 + r] = c[r];
        }
    }
  }
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int row = m0 + (wm * WM + i) * 32 + lane % 32;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = n0 + (wn * WN + j) * 32 + 8 * q + 4 * (lane / 32);
        if (col < N) {
          float s0 = 1.0f, s1 = 1.0f, s2 = 1.0f, s3 = 1.0f;
          if constexpr (B_I8) {
            const f16x4 sc = *reinterpret_cast<const f16x4*>(scales + col);
            s0 = (float)sc[0]; s1 = (float)sc[1]; s2 = (float)sc[2]; s3 = (float)sc[3];
          }
          f32x4 c = {acc[i][j][q * 4 + 0] * s0, acc[i][j][q * 4 + 1] * s1, acc[i][j][q * 4 + 2] * s2,
                     acc[i][j][q * 4 + 3] * s3};
          store4<OutT>(C + (int64_t)row * ldc + col, c[0], c[1], c[2], c[3]);
        }
      }
    }
  }
}

// ---- K % 64 == 0: paired slabs ------------------------------------------------------------------------------
// A K-contiguous operand fetched 32 elements of K at a time touches half of a 128-byte line per row; the other
// half is fetched one slab later, by which time the line has left the vector L1, so every line crosses
// L2 -> L1 twice. Here a stage holds 64 elements of K: each row of a copy is one whole line (8 lanes x 16 bytes),
// the L2 request count halves, and one barrier serves 64 elements of K instead of 32.
constexpr int BK2 = 64;
__device__ __forceinline__ int swz_k2(int row) { return (row >> 1) & 7; }      // row pitch 128 B: 16 rows, 16 slots
// The int8-B kernel reads the same rows with another lane-to-chunk assignment (lane group g takes chunk 2g + step
// instead of 4*step + g); with swz_k2 those reads take twice the cycles in the LDS (measured: 8.3 against 4.6 per
// wave-wide 16-byte read with the LDS saturated). Of the 4096 XOR-linear maps of the row bits this is one of the
// single-bit ones that run both at full rate.
__device__ __forceinline__ int swz_k2i(int row) { return ((row >> 1) & 1) | ((row & 1) << 1) | (row & 4); }
template <bool ALT> __device__ __forceinline__ int swz_k2_sel(int row) { return ALT ? swz_k2i(row) : swz_k2(row); }
// N-contiguous tiles: 32 lanes of a transposing read touch 8 rows (k%4, k/8%2) x 32 bytes of one column block;
// the XOR spreads them over the eight 32-byte slots of 256 bytes of banks. A row's chunks stay whole 128-byte lines.
__device__ __forceinline__ int swz_n2(int k) { return ((k & 3) | (((k >> 3) & 1) << 2)) << 1; }

// Copies are copy_to_lds() buffer loads: rows and column chunks outside the matrix are clamped by the loaders,
// per-lane offsets stay below 2^31 (checked by the launcher).

template <typename T, int ROWS, bool ALT = false>
struct KMajorLoader2 {
  static constexpr int NI = ROWS / 32;              // 8 rows per wave-wide copy, four waves
  int voff[NI];
  int lds_off[NI];
  // row0 + row is clamped to row_max; offsets are relative to row row0 of g
  __device__ __forceinline__ void init(int64_t ld, int row0, int row_max, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * 4 + wave;
      const int row = inst * 8 + lane / 8;
      const int c = (lane % 8) ^ swz_k2_sel<ALT>(row);
      int grow = row0 + row;
      grow = grow < row_max ? grow : row_max;
      voff[j] = (int)(((int64_t)(grow - row0) * ld + c * kChunk) * (int64_t)sizeof(T));
      lds_off[j] = inst * 8 * BK2;
    }
  }
  __device__ __forceinline__ void issue(int j, T* lds, const char* base) const {   // j: an unrolled constant
    if (j < NI) copy_to_lds(base, voff[j], lds + lds_off[j]);
  }
};

template <typename T, int COLS>
struct NMajorLoader2 {
  static constexpr int NI = COLS / 32;              // [64 x COLS] elements, 512 per copy, four waves
  static constexpr int CPR = COLS / kChunk;
  int voff[NI];
  int lds_off[NI];
  // column chunks past col_max are clamped; offsets are relative to column col0 of row 0 of g
  __device__ __forceinline__ void init(int64_t ld, int col0, int col_max, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * 4 + wave;
      const int lin = inst * 64 + lane;
      const int k = lin / CPR;
      const int c = (lin % CPR) ^ swz_n2(k);
      int gcol = col0 + c * kChunk;
      gcol = gcol < col_max ? gcol : col_max;
      voff[j] = (int)(((int64_t)k * ld + (gcol - col0)) * (int64_t)sizeof(T));
      lds_off[j] = inst * 64 * kChunk;
    }
  }
  __device__ __forceinline__ void issue(int j, T* lds, const char* base) const {   // j: an unrolled constant
    if (j < NI) copy_to_lds(base, voff[j], lds + lds_off[j]);
  }
};

template <typename T, bool ALT = false>
__device__ __forceinline__ typename Mfma<T>::Frag read_kmajor2(const T* lds, int row, int chunk) {
  typedef typename Mfma<T>::Frag Frag;
  return *reinterpret_cast<const Frag*>(lds + row * BK2 + ((chunk ^ swz_k2_sel<ALT>(row)) * kChunk));
}

// ds_read_tr16_b64: 16 lanes hand in the addresses of a [4 k x 16 columns] block (lane i: row i/4, columns
// 4*(i%4)..+3) and lane i receives column i's four k values; two of them give a lane 8 consecutive k.
template <typename T, int COLS>
__device__ __forceinline__ typename Mfma<T>::Frag read_nmajor2(const T* lds, int col_tile, int ks, int lane) {
  typedef typename Mfma<T>::Frag Frag;
  constexpr int CPR = COLS / kChunk;
  const int g = lane / 16, i = lane % 16;
  const int n = col_tile + (i & 3) * 4;
  const int kb = ks * 32 + g * 8 + (i >> 2);
  union { i16x4 h[2]; Frag f; } u;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const int k = kb + p * 4;
    const int c = (n / kChunk) ^ swz_n2(k);
    const T* addr = lds + (k * CPR + c) * kChunk + (n % kChunk);
    u.h[p] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(addr));
  }
  return u.f;
}

// Weight-only quantised B: int8 [N,K] rows, 64 bytes per row and slab (four 16-byte chunks, 16 rows per copy),
// kept as int8 in LDS and widened to fp16 in registers, one fragment (8 values of one row) at a time.
// row pitch 64 B. (row >> 2) & 3 also gives every 16 lanes sixteen different slots, but reads at half the rate.
__device__ __forceinline__ int swz_k8(int row) { return (row >> 1) & 3; }
template <int ROWS>
struct I8RowLoader2 {
  static constexpr int NI = ROWS / 64;              // 16 rows per wave-wide copy, four waves
  int voff[NI];
  int lds_off[NI];
  __device__ __forceinline__ void init(int64_t ld, int row0, int row_max, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int inst = j * 4 + wave;
      const int row = inst * 16 + lane / 4;
      const int c = (lane % 4) ^ swz_k8(row);
      int grow = row0 + row;
      grow = grow < row_max ? grow : row_max;
      voff[j] = (int)((int64_t)(grow - row0) * ld + c * 16);
      lds_off[j] = inst * 16 * (BK2 / 4);           // 32-bit words
    }
  }
  // The LDS stage is declared as 32-bit words, not bytes: accesses through a character type may alias anything, and
  // the compiler then holds every fragment read until all copies in flight have landed.
  __device__ __forceinline__ void issue(int j, uint32_t* lds, const char* base) const {   // j: an unrolled constant
    if (j < NI) copy_to_lds(base, voff[j], lds + lds_off[j]);
  }
};
// One 16-byte read per lane and slab: lane (row lane%16, K group g = lane/16) takes bytes [16g, 16g+16) of its row,
// the first 8 for step 0 and the last 8 for step 1; the K slots of an MFMA may be assigned freely as long as A
// uses the same assignment (k = 16g + 8*step + 0..7). (An 8-byte read per step would do, but the compiler then
// holds every such read until all copies in flight have landed.)
__device__ __forceinline__ u32x4 read_i8row(const uint32_t* lds, int row, int kgroup) {
  return *reinterpret_cast<const u32x4*>(lds + row * (BK2 / 4) + ((kgroup ^ swz_k8(row)) * 4));
}
__device__ __forceinline__ f16x8 widen_i8(u32x2 raw) {
  union { uint32_t u[4]; f16x8 f; } r;
  cvt4(raw[0], r.u[0], r.u[1]);
  cvt4(raw[1], r.u[2], r.u[3]);
  return r.f;
}

// The accumulator is tied to the destination in inline assembly: left to the compiler, the 16x16x32 builtin gets
// a destination register of its own and a copy back per instruction. Each accumulator is touched once per 64
// MFMAs, far beyond the instruction's latency; the wait states before the epilogue's first read of an accumulator
// are spent explicitly after the K loop.
template <typename T> struct Mfma16;
template <> struct Mfma16<f16> {
  static __device__ __forceinline__ void run(const f16x8& a, const f16x8& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};
template <> struct Mfma16<bf16> {
  static __device__ __forceinline__ void run(const bf16x8& a, const bf16x8& b, f32x4& c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
};

// Two stages of [tile x 64], MFMA 16x16x32 (on random data the chip runs at its power limit, and this shape
// sustains about 12 % more than 32x32x16 there: it updates a quarter of the accumulators per instruction for half
// the products). A wave owns TM x TN tiles of 16x16 and runs, per paired slab j, two steps of 32 elements of K;
// each step is two phases of TM/2 * TN MFMAs. Fragments of the next step are read while the current one
// multiplies. The copies of slab j+1 are issued in phase 3 of slab j-1 (A) and phase 0 of slab j (B), into the
// stage slab j-1 was read from; the one barrier, between phases 2 and 3, comes after every wave's last read of
// slab j and after all of slab j+1 has landed. NS = 4 stages (small tiles, whose slabs are too short to cover the
// memory latency with one slab of lead) fill the stage of slab j with slab j+4 instead. TAIL: the slab count is not
// a multiple of NS.
// EPI: the kernel adds bias and / or a residual in its epilogue (instantiated apart, so the plain product keeps its
// register allocation).
template <typename T, typename OutT, int WM, int WN, bool TRANS_B, bool TAIL, bool B_I8 = false, int NS = 2,
          bool EPI = false>
__global__ __launch_bounds__(256)
void gemm_kernel_k64(const T* __restrict__ A, const void* __restrict__ Bv, typename OutPtr<OutT, EPI>::type C, int M, int N, int K,
                     int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n,
                     const f16* __restrict__ scales = nullptr, const OutT* __restrict__ bias = nullptr,
                     const OutT* resid = nullptr, int64_t ldr = 0, int out_elems = 0) {
  static_assert(!B_I8 || (TRANS_B && sizeof(T) == 2), "int8 B is [N,K] and multiplies fp16 A");
  const T* B = static_cast<const T*>(Bv);
  typedef typename Mfma<T>::Frag Frag;
  constexpr int BM = 2 * WM * 32, BN = 2 * WN * 32;
  constexpr int TM = 2 * WM, TN = 2 * WN;           // 16x16 tiles per wave
  static_assert(NS == 2 || NS == 4, "two stages, or four for small tiles");
  __shared__ __attribute__((aligned(16))) T a_p0[BM * BK2];
  __shared__ __attribute__((aligned(16))) T a_p1[BM * BK2];
  __shared__ __attribute__((aligned(16))) T a_p2[NS == 4 ? BM * BK2 : 8];
  __shared__ __attribute__((aligned(16))) T a_p3[NS == 4 ? BM * BK2 : 8];
  // int8 B keeps its own element type end to end (copies and reads must name the same LDS objects for the
  // compiler to tell the stage being filled from the stage being read); same bytes, so a wave's result tile fits
  typedef typename std::conditional<B_I8, uint32_t, T>::type BT;
  __shared__ __attribute__((aligned(16))) BT b_p0[BN * BK2 / (B_I8 ? 2 : 1)];
  __shared__ __attribute__((aligned(16))) BT b_p1[BN * BK2 / (B_I8 ? 2 : 1)];
  __shared__ __attribute__((aligned(16))) BT b_p2[NS == 4 ? BN * BK2 / (B_I8 ? 2 : 1) : 8];
  __shared__ __attribute__((aligned(16))) BT b_p3[NS == 4 ? BN * BK2 / (B_I8 ? 2 : 1) : 8];

  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // scalar: LDS destinations stay scalar
  const int wm = wave / 2, wn = wave % 2;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;

  // Epilogue operands are fetched up front, in the accumulators' layout (a lane's four columns of a row: 8 or 16
  // bytes), so their latency passes under the K loop instead of at the end of a tile that has nothing left to
  // overlap it with. Reading before any store of this tile also lets the residual be the output buffer itself.
  typedef typename Run4<OutT>::V EpiRun;
  EpiRun resid_frag[EPI ? TM : 1][EPI ? TN : 1], bias_frag[EPI ? TN : 1];
  if constexpr (EPI) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int col = n0 + (wn * TN + j) * 16 + 4 * (lane / 16);
      col = col < N - 4 ? col : N - 4;                // past the edge: any valid run, those columns are not stored
      if (bias) bias_frag[j] = *reinterpret_cast<const EpiRun*>(bias + col);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        int row = m0 + (wm * TM + i) * 16 + lane % 16;
        row = row < M ? row : M - 1;
        if (resid) resid_frag[i][j] = *reinterpret_cast<const EpiRun*>(resid + (int64_t)row * ldr + col);
      }
    }
  }

  KMajorLoader2<T, BM, B_I8> load_a;
  load_a.init(lda, m0, M - 1, wave, lane);
  KMajorLoader2<T, BN> load_bk;
  NMajorLoader2<T, BN> load_bn;
  I8RowLoader2<BN> load_b8;
  if constexpr (B_I8) load_b8.init(ldb, n0, N - 1, wave, lane);
  else if constexpr (TRANS_B) load_bk.init(ldb, n0, N - 1, wave, lane);
  else load_bn.init(ldb, n0, N - kChunk, wave, lane);     // N % 8 == 0, so n0 <= N - 8
  // uniform bases of this tile's operand panels; slab j adds j * (bytes per 64 elements of K)
  const char* a_base = reinterpret_cast<const char*>(A + (int64_t)m0 * lda);
  const char* b_base = B_I8 ? static_cast<const char*>(Bv) + (int64_t)n0 * ldb
                            : reinterpret_cast<const char*>(TRANS_B ? B + (int64_t)n0 * ldb : B + n0);
  const int64_t a_step = BK2 * (int64_t)sizeof(T);
  const int64_t b_step = B_I8 ? BK2 : (TRANS_B ? BK2 : BK2 * ldb) * (int64_t)sizeof(T);
  constexpr int NLA = BM / 32, NLB = B_I8 ? BN / 64 : BN / 32;

  static_assert(TM == TN && TN >= 4, "a round carries two fragment reads: 2*TM rounds read TM+TN fragments twice");
  auto copy_a = [&](int i, const char* base, T* dst) __attribute__((always_inline)) {
    load_a.issue(i, dst, base);
  };
  auto copy_b = [&](int i, const char* base, BT* dst) __attribute__((always_inline)) {
    if constexpr (B_I8) load_b8.issue(i, dst, base);
    else if constexpr (TRANS_B) load_bk.issue(i, dst, base);
    else load_bn.issue(i, dst, base);
  };
  // fragments of step ks (32 elements of K): lane holds row/column lane%16 of a tile, K group lane/16 (8 elements)
  auto read_a = [&](const T* src, int ks, int i) __attribute__((always_inline)) {
    // int8 B fixes the K slots of a step as k = 16*(lane/16) + 8*step + 0..7 (see read_i8row)
    return read_kmajor2<T, B_I8>(src, (wm * TM + i) * 16 + lane % 16, B_I8 ? 2 * (lane / 16) + ks : ks * 4 + lane / 16);
  };
  auto read_b = [&](const BT* src, int ks, int j) __attribute__((always_inline)) {
    if constexpr (B_I8) return Frag{};              // int8 B is read raw (read_b8) and widened later
    else if constexpr (TRANS_B) return read_kmajor2<T>(src, (wn * TN + j) * 16 + lane % 16, ks * 4 + lane / 16);
    else return read_nmajor2<T, BN>(src, (wn * TN + j) * 16, ks, lane);
  };
  auto read_b8 = [&](const BT* src, int j) __attribute__((always_inline)) {
    if constexpr (B_I8) return read_i8row(src, (wn * TN + j) * 16 + lane % 16, lane / 16);
    else return u32x4{};
  };
  const int KT = K / BK2;
  auto clampj = [&](int j) { return j < KT ? j : KT - 1; };      // past the end: reload the last slab (never used)

  // Copy n of a slab: the NLA copies of A, then the NLB of B.
  constexpr int NL = NLA + NLB;
  auto copy_n = [&](int n, int slab, T* a_dst, BT* b_dst) __attribute__((always_inline)) {
    if constexpr (TRANS_B) {
      if (n < NLA) copy_a(n, a_base + slab * a_step, a_dst);
      else copy_b(n - NLA, b_base + slab * b_step, b_dst);
    } else {
      if (n < NLB) copy_b(n, b_base + slab * b_step, b_dst);
      else copy_a(n - NLB, a_base + slab * a_step, a_dst);
    }
  };
  // Fragment n of a step: the TN of B (every MFMA row needs all of them), then the TM of A in row order.
  u32x4 braw[TN];                                   // int8 B: both steps of a slab as read, before widening
  auto widen_b = [&](int ks, int j, Frag* bf_dst) __attribute__((always_inline)) {
    if constexpr (B_I8) bf_dst[j] = widen_i8(u32x2{braw[j][2 * ks], braw[j][2 * ks + 1]});
  };
  auto read_n = [&](int n, const T* a_src, const BT* b_src, int ks, Frag* af_dst, Frag* bf_dst) __attribute__((always_inline)) {
    if (n < TN) {
      if constexpr (B_I8) {
        if (ks == 0) braw[n] = read_b8(b_src, n);   // once per slab, with the reads of its step 0
      } else {
        bf_dst[n] = read_b(b_src, ks, n);
      }
    } else {
      af_dst[n - TN] = read_a(a_src, ks, n - TN);
    }
  };

  Frag af[2][TM], bf[2][TN];
  // A slab's copies are issued in the window between the barrier that frees their stage and the next barrier:
  // copies_before(w) of them before round w of the window (2*TM rounds). LATE of them fall after the slab boundary,
  // so the prologue leaves slab 1's last LATE copies to slab 0.
  // K-contiguous B: two copies in each of the TM rounds after the barrier (longest lead); N-contiguous B: two in
  // each of the first TM/2 rounds, then one per round, the last TM/2 of them after the slab boundary. Measured on
  // 8192^3 bf16 against five other placements.
  auto copies_before = [](int w) constexpr {
    int sum = 0;
    for (int r = 0; r < w; ++r) {
      if (TRANS_B) sum += 2 * r + 2 <= NL ? 2 : (2 * r < NL ? 1 : 0);
      else sum += r < TM / 2 ? 2 : (r < TM + TM / 2 ? 1 : 0);
    }
    return sum;
  };
  constexpr int LATE = NL - copies_before(TM);
  static_assert(copies_before(2 * TM) == NL, "the window carries all of a slab's copies");
#pragma unroll
  for (int n = 0; n < NL; ++n) copy_n(n, 0, a_p0, b_p0);
  if constexpr (NS == 4) {
#pragma unroll
    for (int n = 0; n < NL; ++n) copy_n(n, clampj(1), a_p1, b_p1);
#pragma unroll
    for (int n = 0; n < NL; ++n) copy_n(n, clampj(2), a_p2, b_p2);
#pragma unroll
    for (int n = 0; n < NL - LATE; ++n) copy_n(n, clampj(3), a_p3, b_p3);
  } else {
#pragma unroll
    for (int n = 0; n < NL - LATE; ++n) copy_n(n, clampj(1), a_p1, b_p1);
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 1) * NL - LATE));  // slab 0 landed
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int n = 0; n < TM + TN; ++n) read_n(n, a_p0, b_p0, 0, af[0], bf[0]);
#pragma unroll
  for (int j = 0; j < TN; ++j) widen_b(0, j, bf[0]);

  // The MFMAs are inline assembly, which the scheduler's group directives do not see, so the issue order is the
  // source order, pinned by full scheduling fences. A slab is 2*TM rounds of TN MFMAs (one row of tiles); a round
  // carries two fragment reads and up to two copies, one after every other MFMA. The barrier sits in the middle:
  // by then every wave has read both steps of this slab, and all of the next slab has landed.
#define HEXMI_FENCE __builtin_amdgcn_sched_barrier(0)
  // cur / nxt / prv: the stages of slabs j, j+1 and j-1 (= j+NS-1; with two stages prv is nxt).
  auto slab = [&](T* acur, BT* bcur, T* anxt, BT* bnxt, T* aprv, BT* bprv, int j) __attribute__((always_inline)) {
    const bool live = !TAIL || j < KT;
    const int j1 = clampj(j + NS - 1), j2 = clampj(j + NS);
#pragma unroll
    for (int q = 0; q < 2 * TM; ++q) {
      const int ks = q / TM, row = q % TM;
      if (q == TM) {
        HEXMI_FENCE;
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((NS - 2) * NL));    // all but slabs j+2 .. j+NS-1 have landed
        __builtin_amdgcn_s_barrier();
        HEXMI_FENCE;
      }
#pragma unroll
      for (int jj = 0; jj < TN / 2; ++jj) {
        if (live) {
          // odd rounds walk the row of tiles backwards: the round boundary then changes one MFMA operand, not both.
          // The kernel runs at the power limit and operand bits that do not toggle are power: +0.6 % at bf16 8192^3
          // and +0.5 % at fp16 4096^3, six alternating runs each on one box, every run of the new order ahead of
          // every run of the old one at 8192^3. (Which of the two operands a round holds fixed makes no difference.)
          const int c0 = (row & 1) ? TN - 1 - 2 * jj : 2 * jj, c1 = (row & 1) ? c0 - 1 : c0 + 1;
          Mfma16<T>::run(bf[ks][c0], af[ks][row], acc[row][c0]);
          Mfma16<T>::run(bf[ks][c1], af[ks][row], acc[row][c1]);
        }
        HEXMI_FENCE;
        // side instructions of slot jj of round q
        if (jj < 2) {
          // fragment reads: first half of the slab reads step 1 of this slab, second half step 0 of the next
          const int n = row * 2 + jj;
          if (ks == 0) read_n(n, acur, bcur, 1, af[1], bf[1]);
          else read_n(n, anxt, bnxt, 0, af[0], bf[0]);
          if constexpr (B_I8) {
            // widen two B fragments per round: step 1 of this slab during its first half (read long ago), step 0
            // of the next slab during the second half, one (small tile) or two rounds after its read
            constexpr int FIRST = TN >= 8 ? 2 : 1;
            const int m = ks == 0 ? 2 * row + jj : 2 * (row - FIRST) + jj;
            if (m >= 0 && m < TN) widen_b(1 - ks, m, bf[1 - ks]);
          }
        }
        constexpr int CSLOT = (TN >= 8 && !TRANS_B) ? 2 : 0;   // first of the two copy slots of a round
        if (jj >= CSLOT && jj < CSLOT + 2) {
          // copies of the window that opened at this slab's barrier (rounds TM..2TM-1, slab j+NS into this slab's
          // stage) and of the window that opened at the previous one (rounds 0.., slab j+NS-1 into the stage of j-1)
          const int c = jj - CSLOT;
          const int w = (q + TM) % (2 * TM);               // round index within its window
          const int lo = copies_before(w), hi = copies_before(w + 1);
          if (lo + c < hi) {
            if (ks == 1) copy_n(lo + c, j2, acur, bcur);
            else copy_n(lo + c, j1, aprv, bprv);
          }
        }
        HEXMI_FENCE;
      }
    }
  };
  for (int j = 0; j < KT; j += NS) {
    if constexpr (NS == 2) {
      slab(a_p0, b_p0, a_p1, b_p1, a_p1, b_p1, j);
      slab(a_p1, b_p1, a_p0, b_p0, a_p0, b_p0, j + 1);
    } else {
      slab(a_p0, b_p0, a_p1, b_p1, a_p3, b_p3, j);
      slab(a_p1, b_p1, a_p2, b_p2, a_p0, b_p0, j + 1);
      slab(a_p2, b_p2, a_p3, b_p3, a_p1, b_p1, j + 2);
      slab(a_p3, b_p3, a_p0, b_p0, a_p2, b_p2, j + 3);
    }
    // The MFMAs are assembly, so the compiler does not count the wait states between the last of them and the
    // first read of an accumulator (19 for the longest matrix instruction). They are spent here, at the end of the
    // last pass and still inside the loop: the register allocator places its accumulator reads at the top of the
    // block that follows the loop, above anything written there.
    if (j + NS >= KT) {
      HEXMI_FENCE;
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
      HEXMI_FENCE;
    }
  }
#undef HEXMI_FENCE
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0));       // drain the trailing copies before the workgroup's LDS goes away

  // acc[i][j][r]: row lane%16 of tile row i, column 4*(lane/16) + r of tile column j
  if constexpr (B_I8) {
    // per-output-channel scales multiply the finished sums
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int col = n0 + (wn * TN + j) * 16 + 4 * (lane / 16);
      col = col < N - 4 ? col : N - 4;              // past the edge: any valid run, those columns are not stored
      const f16x4 sc = *reinterpret_cast<const f16x4*>(scales + col);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] *= (float)sc[r];
    }
  }
  if constexpr (EPI) {
    // bias and residual join the fp32 sums in registers, before their one rounding to the output type
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (bias) acc[i][j][r] += to_f32<OutT>(bias_frag[j][r]);
          if (resid) acc[i][j][r] += to_f32<OutT>(resid_frag[i][j][r]);
        }
  }
  if constexpr (sizeof(OutT) == 2) {
    // (the 256x256 tiles with a guarded last pass sit at the register limit: with this form they would spill)
    const bool by_elements = (WM <= 2 || !TAIL) && out_elems;
    if (ldc % 8 == 0 || by_elements) {
      // 16-bit results go through LDS so that a store instruction writes whole rows of the wave's tile (TN*32
      // contiguous bytes per row) instead of 8-byte pieces of 16 rows. Each wave stages its tile in one of the four
      // operand stages (same size or larger); chunks are XOR-swizzled so both the 8-byte writes and the 16-byte
      // reads spread over the banks.
      // out_elems: the rows of the output start off the 16-byte boundaries (an odd N or leading dimension, an
      // unaligned base): the staged tile leaves in the aligned pieces each row holds, its ends by elements.
      __syncthreads();                                // every wave has finished reading fragments
      OutT* cs = wave == 0 ? reinterpret_cast<OutT*>(a_p0) : wave == 1 ? reinterpret_cast<OutT*>(a_p1)
                 : wave == 2 ? reinterpret_cast<OutT*>(b_p0) : reinterpret_cast<OutT*>(b_p1);
      constexpr int CP = TN * 2;                      // 16-byte chunks per row of the wave's tile
      constexpr int PITCH = TN * 16;                  // elements
      static_assert(TM * 16 * PITCH <= BM * BK2 && TM * 16 * PITCH <= BN * BK2, "a wave's tile fits one stage");
      auto swz = [](int row) { return CP == 16 ? (row & 15) : ((row >> 1) & 7); };
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = i * 16 + lane % 16;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int col = j * 16 + 4 * (lane / 16);
          store4<OutT>(cs + row * PITCH + (((col / kChunk) ^ swz(row)) * kChunk) + col % kChunk, acc[i][j][0],
                       acc[i][j][1], acc[i][j][2], acc[i][j][3]);
        }
      }
      if (by_elements) {
        // A row of C starts anywhere, but most of it is whole 16-byte pieces: a lane gathers the eight elements of
        // one aligned piece from the staged tile (they straddle two of its chunks) and stores them at once, 64 / CP
        // rows per instruction; what a row has before its first boundary and after its last whole piece (up to
        // seven elements each) goes element by element, a lane per row.
        constexpr int W = TN * 16;                    // columns of the wave's tile
        const int gbase = n0 + wn * W;
        const int ncols = N - gbase < W ? (int)(N - gbase) : W;
        const int64_t c_elem = (int64_t)(reinterpret_cast<uintptr_t>(C) / sizeof(OutT));
        auto staged = [&](int row, int col) {
          return cs[row * PITCH + (((col / kChunk) ^ swz(row)) * kChunk) + col % kChunk];
        };
        // columns up to the row's first 16-byte boundary
        auto lead_of = [&](int64_t e0) { return (int)((kChunk - ((c_elem + e0) & (kChunk - 1))) & (kChunk - 1)); };
        constexpr int RPS = 64 / CP;
#pragma unroll 2
        for (int r0 = 0; r0 < TM * 16; r0 += RPS) {
          const int row = r0 + lane / CP, q = lane % CP;
          const int grow = m0 + wm * TM * 16 + row;
          const int64_t e0 = (int64_t)grow * ldc + gbase;
          const int c0 = lead_of(e0) + kChunk * q;
          if (grow < M && c0 + kChunk <= ncols) {
            __attribute__((aligned(16))) OutT o[kChunk];
#pragma unroll
            for (int i = 0; i < kChunk; ++i) o[i] = staged(row, c0 + i);
            __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(o), reinterpret_cast<u32x4*>(C + e0 + c0));
          }
        }
#pragma unroll 1
        for (int r0 = 0; r0 < TM * 16; r0 += 64) {
          const int row = r0 + lane;
          const int grow = m0 + wm * TM * 16 + row;
          if (row < TM * 16 && grow < M && ncols > 0) {
            const int64_t e0 = (int64_t)grow * ldc + gbase;
            const int lead = lead_of(e0);
            const int head = lead < ncols ? lead : ncols;
            const int tail = ncols > lead ? lead + ((ncols - lead) & ~(kChunk - 1)) : ncols;
            // every read ahead of the first store, the stores under masks (one read and one store per turn of a loop
            // would put their latencies end to end)
            OutT hv[kChunk - 1], tv[kChunk - 1];
#pragma unroll
            for (int k = 0; k < kChunk - 1; ++k) {
              hv[k] = staged(row, k);
              tv[k] = staged(row, tail + k < W ? tail + k : W - 1);
            }
#pragma unroll
            for (int k = 0; k < kChunk - 1; ++k) {
              if (k < head) C[e0 + k] = hv[k];
              if (tail + k < ncols) C[e0 + tail + k] = tv[k];
            }
          }
        }
        return;
      }
      constexpr int RPI = 64 / CP;                    // rows per store instruction
#pragma unroll
      for (int r0 = 0; r0 < TM * 16; r0 += RPI) {
        const int row = r0 + lane / CP, c = lane % CP;
        const u32x4 v = *reinterpret_cast<const u32x4*>(cs + row * PITCH + ((c ^ swz(row)) * kChunk));
        const int grow = m0 + wm * TM * 16 + row, gcol = n0 + wn * TN * 16 + c * kChunk;
        // non-temporal: C is not read again, and the operand panels other tiles still need stay in the caches
        // (bf16 8192^3: 0.617 -> 0.632 of peak, A/B on one box; 4096^3 unchanged)
        if (grow < M && gcol < N) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(C + (int64_t)grow * ldc + gcol));
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = m0 + (wm * TM + i) * 16 + lane % 16;
    if (row >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = n0 + (wn * TN + j) * 16 + 4 * (lane / 16);
      if (col < N)
        store4<OutT>(C + (int64_t)row * ldc + col, acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
    }
  }
}

// Any shape, any alignment: what the kernels above do not take -- operand rows that do not start on 16-byte
// boundaries (an odd leading dimension, a base that is a view into a larger tensor), K not a multiple of 8, B given as
// [K,N] with a ragged N. 128x128 tiles, four waves of 2x2 MFMA tiles, the LDS layouts and fragment reads of
// gemm_kernel; but the slabs come through registers: 16-byte global loads at whatever alignment the rows have (the
// hardware takes them at 2-byte alignment; the global -> LDS copy path is kept for aligned chunks), issued for slab
// kt + 1 before slab kt is multiplied and written to the other LDS stage after it, one barrier per slab. A chunk that
// reaches past K (or, B as [K,N], past N) is put together from guarded element loads with zeros behind the edge; rows
// past M (and past N, B as [N,K]) are clamped, their products never stored. The result leaves in rows through LDS
// (store_tile_by_rows). About 0.5 PFLOP/s where the one-MFMA-per-barrier kernel this replaces ran 0.07.
template <typename T>
__device__ __forceinline__ u32x4 load_chunk_any(const T* p, int valid) {
  u32x4 v;
  if (valid >= kChunk) {
    __builtin_memcpy(&v, p, 16);                    // alignment of T only: one global_load_dwordx4
  } else {
    unsigned short e[kChunk];
#pragma unroll
    for (int t = 0; t < kChunk; ++t) e[t] = t < valid ? reinterpret_cast<const unsigned short*>(p)[t] : (unsigned short)0;
#pragma unroll
    for (int t = 0; t < 4; ++t) v[t] = (unsigned)e[2 * t] | ((unsigned)e[2 * t + 1] << 16);
  }
  return v;
}

// Eight int8 weights (any alignment, `valid` of them inside the row) minus the zero point, as eight fp16: exact.
__device__ __forceinline__ u32x4 load_chunk_i8(const int8_t* p, int valid, int zero_point) {
  int8_t b[kChunk];
  if (valid >= kChunk) {
    __builtin_memcpy(b, p, kChunk);                 // one global_load_dwordx2
  } else {
#pragma unroll
    for (int t = 0; t < kChunk; ++t) b[t] = t < valid ? p[t] : (int8_t)0;
  }
  union { f16 h[kChunk]; u32x4 v; } u;
#pragma unroll
  for (int t = 0; t < kChunk; ++t) u.h[t] = t < valid ? (f16)(float)((int)b[t] - zero_point) : (f16)0.0f;
  return u.v;
}

// B_I8: B is int8 [N,K] (needs TRANS_B, fp16 A and C): (W - zero_point) is formed in fp16 on the way into LDS and the
// finished sums are multiplied by scales[column] (one scale and zero point for the tensor with per_tensor).
template <typename T, typename OutT, bool TRANS_B, bool B_I8 = false>
__global__ __launch_bounds__(256)
void gemm_kernel_any(const T* __restrict__ A, const void* __restrict__ Bv, OutT* C, int M, int N, int K, int64_t lda,
                     int64_t ldb, int64_t ldc, int tiles_m, int tiles_n, const OutT* __restrict__ bias = nullptr,
                     const OutT* resid = nullptr, int64_t ldr = 0, const f16* __restrict__ scales = nullptr,
                     const int8_t* __restrict__ zero_points = nullptr, int per_tensor = 0) {
  static_assert(sizeof(T) == 2, "16-bit operands");
  static_assert(!B_I8 || (TRANS_B && std::is_same<T, f16>::value), "int8 B is [N,K] and multiplies fp16 A");
  const T* B = static_cast<const T*>(Bv);
  const int8_t* B8 = static_cast<const int8_t*>(Bv);
  typedef typename Mfma<T>::Frag Frag;
  constexpr int WM = 2, WN = 2, NW = 4, BM = 128, BN = 128;
  __shared__ __attribute__((aligned(16))) T a_s[2][BM * BK];
  __shared__ __attribute__((aligned(16))) T b_s[2][BN * BK];
  __shared__ __attribute__((aligned(16))) OutT c_s[RaggedStage<OutT>::kRows * RaggedStage<OutT>::pitch(BN)];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / 2, wn = wave % 2;
  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Two chunks of each operand per thread and slab. K-contiguous tile: chunk e -> row e / 4, source chunk e % 4.
  // [K,N] tile: chunk e -> slab row e / 16, source chunk e % 16. LDS positions as in KMajorLoader / NMajorLoader.
  const T* a_ptr[2];
  const T* b_ptr[2];
  const int8_t* b8_ptr[2];
  int a_k[2], b_k[2], a_pos[2], b_pos[2], b_valid_n[2], b_zero[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int e = j * 256 + tid;
    {
      const int row = e / 4, c = e % 4;
      int grow = m0 + row;
      grow = grow < M - 1 ? grow : M - 1;
      a_ptr[j] = A + (int64_t)grow * lda + c * kChunk;
      a_k[j] = c * kChunk;
      a_pos[j] = row * BK + ((c ^ swz_k(row)) * kChunk);
    }
    if constexpr (TRANS_B) {
      const int row = e / 4, c = e % 4;
      int grow = n0 + row;
      grow = grow < N - 1 ? grow : N - 1;
      if constexpr (B_I8) b8_ptr[j] = B8 + (int64_t)grow * ldb + c * kChunk;
      else b_ptr[j] = B + (int64_t)grow * ldb + c * kChunk;
      b_k[j] = c * kChunk;
      b_pos[j] = row * BK + ((c ^ swz_k(row)) * kChunk);
      b_valid_n[j] = kChunk;
      b_zero[j] = B_I8 && zero_points ? (int)zero_points[per_tensor ? 0 : grow] : 0;
    } else {
      constexpr int CPR = BN / kChunk;
      const int k = e / CPR, c = e % CPR;
      const int gcol = n0 + c * kChunk;
      b_valid_n[j] = gcol >= N ? 0 : (N - gcol < kChunk ? N - gcol : kChunk);   // columns of this chunk inside the matrix
      b_ptr[j] = B + (int64_t)k * ldb + (gcol < N ? gcol : 0);
      b_k[j] = k;
      b_pos[j] = (k * CPR + (c ^ swz_n(k))) * kChunk;
    }
  }
  u32x4 ra[2], rb[2];
  auto fetch = [&](int kt) {
    const int k0 = kt * BK;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int left = K - (k0 + a_k[j]);                    // elements of this chunk before the end of K
      ra[j] = load_chunk_any<T>(a_ptr[j] + k0, left < 0 ? 0 : left);
      if constexpr (B_I8) {
        const int leftb = K - (k0 + b_k[j]);
        rb[j] = load_chunk_i8(b8_ptr[j] + k0, leftb < 0 ? 0 : leftb, b_zero[j]);
      } else if constexpr (TRANS_B) {
        const int leftb = K - (k0 + b_k[j]);
        rb[j] = load_chunk_any<T>(b_ptr[j] + k0, leftb < 0 ? 0 : leftb);
      } else {
        rb[j] = load_chunk_any<T>(b_ptr[j] + (int64_t)k0 * ldb, k0 + b_k[j] < K ? b_valid_n[j] : 0);
      }
    }
  };
  auto stash = [&](int stage) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      *reinterpret_cast<u32x4*>(&a_s[stage][a_pos[j]]) = ra[j];
      *reinterpret_cast<u32x4*>(&b_s[stage][b_pos[j]]) = rb[j];
    }
  };
  const int KT = (K + BK - 1) / BK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt & 1;
    if (kt + 1 < KT) fetch(kt + 1);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      Frag af[WM], bf[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) af[i] = read_kmajor<T>(a_s[stage], (wm * WM + i) * 32 + lane % 32, ks * 2 + lane / 32);
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        if constexpr (TRANS_B) bf[j] = read_kmajor<T>(b_s[stage], (wn * WN + j) * 32 + lane % 32, ks * 2 + lane / 32);
        else bf[j] = read_nmajor<T, BN>(b_s[stage], (wn * WN + j) * 32, ks, lane);
      }
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = Mfma<T>::run(bf[j], af[i], acc[i][j]);
    }
    if (kt + 1 < KT) stash(stage ^ 1);
    __syncthreads();
  }
  store_tile_by_rows<OutT, WM, WN, NW, BM, BN>(acc, c_s, C, ldc, bias, resid, ldr, M, N, m0, n0, wm, wn, wave, lane,
                                               B_I8 ? scales : nullptr, per_tensor);
}

// Up to eight activation rows against weights given as [N,K] (x @ W^T, a decode step): the product is a stream of
// the weights at the HBM rate, and tiles of 128 columns would leave most CUs without work (N = K = 4096: 32 tiles,
// 24 us where the 32 MB of weights take 6). One wave per output channel, eight per workgroup: the wave reads its
// weight row 16 bytes per lane (non-temporal, four chunks in flight), the activation rows come from LDS where the
// workgroup staged 2048 columns of them, products accumulate in fp32 (v_dot2) and a butterfly sums the lanes.
// K % 8 == 0, rows on 16-byte boundaries.
template <typename T> struct Dot8;
template <> struct Dot8<f16> {
  static __device__ __forceinline__ float run(const u32x4& w, const u32x4& a, float acc) {
    const f16x8 wf = __builtin_bit_cast(f16x8, w), af = __builtin_bit_cast(f16x8, a);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc = __builtin_amdgcn_fdot2(f16x2{wf[2 * e], wf[2 * e + 1]}, f16x2{af[2 * e], af[2 * e + 1]}, acc, false);
    return acc;
  }
};
template <> struct Dot8<bf16> {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ float run(const u32x4& w, const u32x4& a, float acc) {
    const bf16x8 wf = __builtin_bit_cast(bf16x8, w), af = __builtin_bit_cast(bf16x8, a);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2_t{wf[2 * e], wf[2 * e + 1]}, bf16x2_t{af[2 * e], af[2 * e + 1]}, acc, false);
    return acc;
  }
};

constexpr int kGemvWaves = 8, kGemvBlockK = 2048;

// RPW: output channels per wave (a chunk of activations read from LDS then serves RPW weight rows; measured, it did
// not pay: see the launch).
template <typename T, typename OutT, int MR, int NW = kGemvWaves, int RPW = 1>
__global__ __launch_bounds__(NW * 64)
void gemv_nt_kernel(const T* __restrict__ A, const T* __restrict__ W, OutT* C, int M, int N, int K, int64_t lda,
                    int64_t ldb, int64_t ldc, const OutT* __restrict__ bias, const OutT* resid, int64_t ldr) {
  constexpr int KB = kGemvBlockK, CPB = KB / kChunk;  // chunks per row of a staged block
  constexpr int CPL = CPB / kWave;                    // chunks per lane, row and block
  __shared__ __attribute__((aligned(16))) T a_s[MR][KB];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int n_first = (blockIdx.x * NW + wave) * RPW;
  const T* wrow[RPW];
#pragma unroll
  for (int q = 0; q < RPW; ++q)                        // past the end: the last channel again, not stored
    wrow[q] = W + (int64_t)(n_first + q < N ? n_first + q : N - 1) * ldb;
  float acc[MR][RPW];
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int q = 0; q < RPW; ++q) acc[m][q] = 0.0f;
  for (int kb = 0; kb < K; kb += KB) {
    const int kn = K - kb < KB ? K - kb : KB;           // columns of this block, a multiple of 8
    // the weight chunks of this block first: they come from HBM, the activations below from L2
    u32x4 wv[RPW][CPL];
#pragma unroll
    for (int q = 0; q < RPW; ++q)
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        const int k = (j * kWave + lane) * kChunk;
        wv[q][j] = k < kn ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[q] + kb + k)) : u32x4{0u, 0u, 0u, 0u};
      }
    __syncthreads();                                    // every wave has read the block before
    for (int c = threadIdx.x; c < MR * CPB; c += NW * 64) {
      const int m = c / CPB, k = (c % CPB) * kChunk;
      if (k < kn)
        *reinterpret_cast<u32x4*>(&a_s[m][k]) =
            *reinterpret_cast<const u32x4*>(A + (int64_t)(m < M ? m : M - 1) * lda + kb + k);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
      const int k = (j * kWave + lane) * kChunk;
      if (k < kn) {
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const u32x4 av = *reinterpret_cast<const u32x4*>(&a_s[m][k]);
#pragma unroll
          for (int q = 0; q < RPW; ++q) acc[m][q] = Dot8<T>::run(wv[q][j], av, acc[m][q]);
        }
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int q = 0; q < RPW; ++q) {
      float sum = wave_sum(acc[m][q]);
      const int n = n_first + q;
      if (lane == 0 && n < N && m < M) {
        if (bias) sum += to_f32<OutT>(bias[n]);
        if (resid) sum += to_f32<OutT>(resid[(int64_t)m * ldr + n]);
        C[(int64_t)m * ldc + n] = from_f32<OutT>(sum);
      }
    }
}

// Nine to sixty-four rows against [N,K] weights: still a stream of the weights, now on the matrix cores. One workgroup
// of four waves per tile of 16 output channels (N / 16 workgroups where 128-column tiles would be N / 128); the waves
// split K four ways in runs of whole 128-byte lines and their partial tiles meet in LDS. A lane's 16-byte weight load
// is its MFMA 16x16x32 operand as it stands (channel lane % 16, eight k from 8 * (lane / 16) on), all loads of a round
// issued before the first MFMA; the activation fragments come through L1 / L2. K % 32 == 0, rows on 16-byte
// boundaries. MT: 16-row tiles of activations.
template <typename T> struct Mfma16Builtin;
template <> struct Mfma16Builtin<f16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& w, const u32x4& a, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w), __builtin_bit_cast(f16x8, a), c, 0, 0, 0);
  }
};
template <> struct Mfma16Builtin<bf16> {
  static __device__ __forceinline__ f32x4 run(const u32x4& w, const u32x4& a, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, a), c, 0, 0, 0);
  }
};

template <typename T, typename OutT, int MT>
__global__ __launch_bounds__(256)
void gemm_nt_skinny_kernel(const T* __restrict__ A, const T* __restrict__ W, OutT* C, int M, int N, int K, int64_t lda,
                           int64_t ldb, int64_t ldc, const OutT* __restrict__ bias, const OutT* resid, int64_t ldr) {
  constexpr int NWV = 4;
  __shared__ __attribute__((aligned(16))) float red[NWV * MT * 256];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int r16 = lane % 16, kg = lane / 16;
  const int tile = blockIdx.x;
  const int n = tile * 16 + r16;
  const T* wrow = W + (int64_t)(n < N ? n : N - 1) * ldb + kg * kChunk;
  const int steps = K / 32;
  const int per_wave = (((steps + NWV - 1) / NWV) + 1) & ~1;      // an even number of 64-byte steps: whole lines
  const int s_begin = wave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;
  const T* arow[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int gm = t * 16 + r16;
    arow[t] = A + (int64_t)(gm < M ? gm : M - 1) * lda + kg * kChunk;   // past the end: the last row, not stored
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  constexpr int U = MT == 1 ? 8 : (MT == 2 ? 4 : 2);
  for (int s0 = s_begin; s0 < s_end; s0 += U) {
    u32x4 wv[U], av[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      wv[u] = u32x4{0u, 0u, 0u, 0u};
      if (s0 + u < s_end) wv[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow + (int64_t)(s0 + u) * 32));
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        av[u][t] = u32x4{0u, 0u, 0u, 0u};
        if (s0 + u < s_end) av[u][t] = *reinterpret_cast<const u32x4*>(arow[t] + (int64_t)(s0 + u) * 32);
      }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = Mfma16Builtin<T>::run(wv[u], av[u][t], acc[t]);   // a skipped step is zeros
  }
  // D[i = channel][j = activation row]: a lane holds row lane % 16, channels 4 * (lane / 16) + 0 .. 3
#pragma unroll
  for (int t = 0; t < MT; ++t) *reinterpret_cast<f32x4*>(red + ((wave * MT + t) * 64 + lane) * 4) = acc[t];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MT * 64; idx += 256) {
    const int t = idx / 64, l = idx % 64;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < NWV; ++w) sum += *reinterpret_cast<const f32x4*>(red + ((w * MT + t) * 64 + l) * 4);
    const int gm = t * 16 + l % 16;
    const int gn = tile * 16 + (l / 16) * 4;
    if (gm < M) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (gn + e < N) {
          float v = sum[e];
          if (bias) v += to_f32<OutT>(bias[gn + e]);
          if (resid) v += to_f32<OutT>(resid[(int64_t)gm * ldr + gn + e]);
          C[(int64_t)gm * ldc + gn + e] = from_f32<OutT>(v);
        }
    }
  }
}

// fp32 inputs (the reference's torch-mlir graphs multiply fp32 matrices, e.g.
// test/python/torch-mlir/test_add_matmul_softmax.py:25-29) whose shape or alignment the matrix-core kernel of
// gemm_f32.hip does not take: 64x64 tile, K in steps of 16 through LDS, every thread a 4x4 block of fp32 FMAs.
// Any shape.
template <bool TRANS_B>
__global__ __launch_bounds__(256)
void gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ B, float* C, int M, int N,
                     int K, int64_t lda, int64_t ldb, int64_t ldc, const float* __restrict__ bias = nullptr,
                     const float* resid = nullptr, int64_t ldr = 0) {
  constexpr int TB = 64, TK = 16;
  __shared__ float a_s[TK][TB + 4];                  // [k][m]
  __shared__ float b_s[TK][TB + 4];                  // [k][n]
  const int m0 = blockIdx.y * TB, n0 = blockIdx.x * TB;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;   // thread owns rows ty*4.., columns tx*4..
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += TK) {
    __syncthreads();
    for (int e = threadIdx.x; e < TB * TK; e += 256) {
      {
        const int r = e / TK, k = e % TK;            // A: consecutive threads walk k (contiguous in memory)
        const int gm = m0 + r, gk = k0 + k;
        a_s[k][r] = (gm < M && gk < K) ? A[(int64_t)gm * lda + gk] : 0.0f;
      }
      if (TRANS_B) {
        const int r = e / TK, k = e % TK;            // B[n][k]
        const int gn = n0 + r, gk = k0 + k;
        b_s[k][r] = (gn < N && gk < K) ? B[(int64_t)gn * ldb + gk] : 0.0f;
      } else {
        const int k = e / TB, c = e % TB;            // B[k][n]: consecutive threads walk n
        const int gn = n0 + c, gk = k0 + k;
        b_s[k][c] = (gn < N && gk < K) ? B[(int64_t)gk * ldb + gn] : 0.0f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = b_s[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn < N) {
        float c = acc[i][j];
        if (bias) c += bias[gn];
        if (resid) c += resid[(int64_t)gm * ldr + gn];
        C[(int64_t)gm * ldc + gn] = c;
      }
    }
  }
}

int launch_f32(bool trans_b, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
               int64_t ldb, int64_t ldc, hipStream_t s, const void* bias_v = nullptr, const void* resid_v = nullptr,
               int64_t ldr = 0) {
  const float* a = static_cast<const float*>(A);
  const float* b = static_cast<const float*>(B);
  float* c = static_cast<float*>(C);
  const float* bias = static_cast<const float*>(bias_v);
  const float* resid = static_cast<const float*>(resid_v);
  int status = HEXMI_OK;
  // matrix cores (their kernel has no epilogue operands: a product with bias or residual takes the FMA kernel)
  if (!bias && !resid && gemm_f32_mfma(trans_b, a, b, c, M, N, K, lda, ldb, ldc, s, &status)) return status;
  dim3 grid((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64));
  if (grid.y > 65535) return HEXMI_ENOTSUP;
  if (trans_b)
    hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, dim3(256), 0, s, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, bias,
                       resid, ldr);
  else
    hipLaunchKernelGGL(gemm_f32_kernel<false>, grid, dim3(256), 0, s, a, b, c, (int)M, (int)N, (int)K, lda, ldb, ldc, bias,
                       resid, ldr);
  return launch_status();
}

// out_elems: 16-bit results leave the paired-slab kernel one element per lane (the caller has checked that this
// kernel takes the product: K % 64 == 0, short rows, no bias or residual).
template <typename T, typename OutT, int WM, int WN, bool TRANS_B, int NWN = 2>
int launch_tiled(const T* A, const T* B, OutT* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                 int64_t ldc, hipStream_t s, const OutT* bias, const OutT* resid, int64_t ldr, int out_elems = 0) {
  constexpr int BM = 2 * WM * 32, BN = NWN * WN * 32;
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  // K % 64 == 0: the paired-slab kernel; its per-lane copy offsets (up to 256 rows, or 64 rows of K) must stay
  // below 2^31 bytes
  if (NWN == 2 && K % BK2 == 0 && lda < (1 << 21) && ldb < (1 << 21)) {
    constexpr int NS = WM <= 2 ? 4 : 2;            // small tiles: four stages (their slabs are short)
    if constexpr (WM == 2 && WN == 2) {
      if (bias || resid) {                          // the instantiations that carry the epilogue operands
        if ((K / BK2) % NS == 0)
          hipLaunchKernelGGL((gemm_kernel_k64<T, OutT, WM, WN, TRANS_B, false, false, NS, true>),
                             dim3(tiles_m * tiles_n), dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc,
                             tiles_m, tiles_n, nullptr, bias, resid, ldr);
        else
          hipLaunchKernelGGL((gemm_kernel_k64<T, OutT, WM, WN, TRANS_B, true, false, NS, true>),
                             dim3(tiles_m * tiles_n), dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc,
                             tiles_m, tiles_n, nullptr, bias, resid, ldr);
        return launch_status();
      }
    }
    if ((K / BK2) % NS == 0)
      hipLaunchKernelGGL((gemm_kernel_k64<T, OutT, WM, WN, TRANS_B, false, false, NS>), dim3(tiles_m * tiles_n),
                         dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, tiles_m, tiles_n, nullptr,
                         nullptr, nullptr, 0, out_elems);
    else
      hipLaunchKernelGGL((gemm_kernel_k64<T, OutT, WM, WN, TRANS_B, true, false, NS>), dim3(tiles_m * tiles_n),
                         dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, tiles_m, tiles_n, nullptr,
                         nullptr, nullptr, 0, out_elems);
    return launch_status();
  }
  if (out_elems) return HEXMI_ENOTSUP;             // only the paired-slab kernel has that epilogue
  if constexpr (WM == 2 && WN == 2) {
    if (bias || resid) {
      hipLaunchKernelGGL((gemm_kernel<T, OutT, WM, WN, TRANS_B, true, false, NWN, true>), dim3(tiles_m * tiles_n),
                         dim3(NWN * 128), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, tiles_m, tiles_n, nullptr,
                         bias, resid, ldr);
      return launch_status();
    }
  }
  if ((K / BK) % 4 == 0)
    hipLaunchKernelGGL((gemm_kernel<T, OutT, WM, WN, TRANS_B, false, false, NWN>), dim3(tiles_m * tiles_n),
                       dim3(NWN * 128), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, tiles_m, tiles_n);
  else
    hipLaunchKernelGGL((gemm_kernel<T, OutT, WM, WN, TRANS_B, true, false, NWN>), dim3(tiles_m * tiles_n),
                       dim3(NWN * 128), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, tiles_m, tiles_n);
  return launch_status();
}

// 256 x 256 or 128 x 128 tiles. Either kind runs one workgroup per CU at a time, so a launch is whole rounds over
// the CUs and the last round may be nearly empty. With every round full the large tiles run about 1.3 times the
// rate of the small ones (fp16 K = 4096: 1.4 against 1.08 PFLOP/s; int8 weights: 1.2 against 0.93), and a round
// that is not full runs its tiles somewhat faster: the large tiles are taken when 1.48 times the fill of their
// rounds is at least the fill of the small tiles' rounds. (fp16, K = 4096, 256 CUs: 128 large tiles 825 TFLOP/s
// against 1074 with small ones, 289 tiles 920 against 1019, 192 tiles 1152 against 1077, 324 tiles 1020 against 965;
// int8 weights, N = 11008: M = 512 518 against 680, M = 768 739 against 687.)
inline bool prefer_large_tiles(int64_t M, int64_t N) {
  const int64_t cus = hexmi_num_cus();
  if (cus <= 0) return false;
  const int64_t big = ((M + 255) / 256) * ((N + 255) / 256), small = ((M + 127) / 128) * ((N + 127) / 128);
  const int64_t rounds_big = (big + cus - 1) / cus, rounds_small = (small + cus - 1) / cus;
  if (big > (int64_t)1 << 40) return true;
  return 148 * big * rounds_small >= 100 * small * rounds_big;
}

template <typename T, typename OutT, bool TRANS_B>
int dispatch_gemm(const void* Av, const void* Bv, void* Cv, int64_t M, int64_t N, int64_t K, int64_t lda,
                  int64_t ldb, int64_t ldc, hipStream_t s, const void* bias_v, const void* resid_v, int64_t ldr) {
  const T* A = static_cast<const T*>(Av);
  const T* B = static_cast<const T*>(Bv);
  OutT* C = static_cast<OutT*>(Cv);
  const OutT* bias = static_cast<const OutT*>(bias_v);
  const OutT* resid = static_cast<const OutT*>(resid_v);
  // The tiled kernels copy 16-byte chunks and clamp (never mask) rows / column chunks, so they need whole
  // chunks: K % 32 == 0, leading dimensions and N multiples of 8 elements, 16-byte aligned bases. Their epilogue
  // reads bias and residual in runs of four columns.
  const size_t run = 4 * sizeof(OutT);
  // a few rows against [N,K] weights: the weight stream (see gemv_nt_kernel)
  // (Every workgroup stages the activation rows it multiplies, so their traffic grows with the rows while the
  // weights' does not: up to two rows always, up to four from K = 1024, up to eight from K = 2048 on -- N = 50264,
  // K = 768: 14.6 against 23 us on the tiles at one row, 32 against 23 at eight. Nine to sixteen rows as two passes
  // of eight measured 21.5 against 24 us at N = K = 4096 but 48 against 26 at N = 11008: not taken.)
  if (TRANS_B && (M <= 2 || (M <= 4 && K >= 1024) || (M <= 8 && K >= 2048)) && N >= 64 && K % kChunk == 0 &&
      lda % 8 == 0 && ldb % 8 == 0 && aligned_to(A, 16) && aligned_to(B, 16)) {
#define HEXMI_GEMV(MR, NW, RPW) \
  hipLaunchKernelGGL((gemv_nt_kernel<T, OutT, MR, NW, RPW>), dim3((unsigned)((N + NW * RPW - 1) / (NW * RPW))), dim3(NW * 64), 0, s, \
                     A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, bias, resid, ldr)
    // one channel per wave throughout: two for four rows measured equal to slower (N = 4096, K = 11008: 22.2 against
    // 19.9 us), four for eight rows 38 against 22.5 us at N = 11008 (130 registers, four strided rows per load
    // group); sixteen waves share the staged rows from five rows on (24 -> 22.5 us)
    if (M == 1) HEXMI_GEMV(1, 8, 1); else if (M == 2) HEXMI_GEMV(2, 8, 1); else if (M <= 4) HEXMI_GEMV(4, 8, 1);
    else HEXMI_GEMV(8, 16, 1);
#undef HEXMI_GEMV
    return launch_status();
  }
  // Every workgroup of the skinny kernel pulls all M x K activations through L2, N / 16 times over in total, where
  // the tiles walk K with N / 128 workgroups: it wins while N is near sixteen channels per CU or K is long. Both
  // sides as fitted on 256 CUs, in microseconds (N = K = 4096: 12.1 / 15.4 / 22.3 at 16 / 32 / 64 rows against
  // 24 on the tiles; N = 4096, K = 11008: 27 / 36 / 56 against 57; N = 11008, K = 4096: 28 / 39 / 63 against 26).
  const double nk = (double)N * (double)K;
  const double skinny_us = 3.0 + 2.0 * nk / 6.0e6 + 1.27e-8 * nk * (double)M;
  const double tiles_us = std::max(23.0, 4.0 + 5.2e-3 * (double)K * (double)((N + 128 * 512 - 1) / (128 * 512)));
  if (TRANS_B && M <= 64 && N >= 64 && K % 32 == 0 && lda % 8 == 0 && ldb % 8 == 0 && aligned_to(A, 16) &&
      aligned_to(B, 16) && skinny_us < 0.9 * tiles_us) {
    const dim3 grid((unsigned)((N + 15) / 16));
#define HEXMI_SKINNY(MT) \
  hipLaunchKernelGGL((gemm_nt_skinny_kernel<T, OutT, MT>), grid, dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, \
                     bias, resid, ldr)
    if (M <= 16) HEXMI_SKINNY(1); else if (M <= 32) HEXMI_SKINNY(2); else HEXMI_SKINNY(4);
#undef HEXMI_SKINNY
    return launch_status();
  }
  const bool fast = K % BK == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && N % 8 == 0 && N >= 8 &&
                    aligned_to(A, 16) && aligned_to(B, 16) && aligned_to(C, 16) && (!bias || aligned_to(bias, run)) &&
                    (!resid || (aligned_to(resid, run) && ldr % 4 == 0));
  if (fast) {
    const bool large = prefer_large_tiles(M, N);
    // the large-tile kernels sit at the register limit and carry no epilogue operands: a product with bias or
    // residual runs on the 128x128 tiles at any size
    if (large && !bias && !resid)
      return launch_tiled<T, OutT, 4, 4, TRANS_B>(A, B, C, M, N, K, lda, ldb, ldc, s, nullptr, nullptr, 0);
    return launch_tiled<T, OutT, 2, 2, TRANS_B>(A, B, C, M, N, K, lda, ldb, ldc, s, bias, resid, ldr);
  }
  // Whole 16-byte chunks on the operand side only (K % 8 == 0; B given as [K,N] also N % 8 == 0): the 128x128 tiles
  // with a masked last slab, and an output side that may be anything ([N,K] weights with an odd N, such as a
  // vocabulary of 50257, land here: 1.0 PFLOP/s against 0.1 on the generic kernel below).
  const bool chunks = K % kChunk == 0 && lda % 8 == 0 && ldb % 8 == 0 && aligned_to(A, 16) && aligned_to(B, 16) &&
                      (TRANS_B || (N % 8 == 0 && N >= 8));
  // ... and with whole 64-wide slabs, a 16-bit result and no epilogue operands the paired-slab kernels take it, their
  // staged tiles leaving element by element
  if (chunks && sizeof(OutT) == 2 && K % BK2 == 0 && lda < (1 << 21) && ldb < (1 << 21) && !bias && !resid) {
    if (prefer_large_tiles(M, N) && (K / BK2) % 2 == 0)      // the 256x256 form without a guarded last pass only
      return launch_tiled<T, OutT, 4, 4, TRANS_B>(A, B, C, M, N, K, lda, ldb, ldc, s, nullptr, nullptr, 0, 1);
    return launch_tiled<T, OutT, 2, 2, TRANS_B>(A, B, C, M, N, K, lda, ldb, ldc, s, nullptr, nullptr, 0, 1);
  }
  if (chunks) {
    const bool runs = N % 4 == 0 && N >= 4 && ldc % 4 == 0 && aligned_to(C, run) && (!bias || aligned_to(bias, run)) &&
                      (!resid || (aligned_to(resid, run) && ldr % 4 == 0));
    const int64_t tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
    if (tiles_m * tiles_n > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((gemm_kernel<T, OutT, 2, 2, TRANS_B, true, false, 2, true, true>), dim3((unsigned)(tiles_m * tiles_n)),
                       dim3(256), 0, s, A, B, C, (int)M, (int)N, (int)K, lda, ldb, ldc, (int)tiles_m, (int)tiles_n, nullptr,
                       bias, resid, ldr, runs ? 1 : 0);
    return launch_status();
  }
  const int64_t tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
  if (tiles_m * tiles_n > 0x7fffffff || K > 0x7fffffff - 64) return HEXMI_ENOTSUP;
  hipLaunchKernelGGL((gemm_kernel_any<T, OutT, TRANS_B>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, s, A, B, C,
                     (int)M, (int)N, (int)K, lda, ldb, ldc, (int)tiles_m, (int)tiles_n, bias, resid, ldr);
  return launch_status();
}

template <typename T, typename OutT>
int dispatch_trans(bool trans_b, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K, int64_t lda,
                   int64_t ldb, int64_t ldc, hipStream_t s, const void* bias, const void* resid, int64_t ldr) {
  return trans_b ? dispatch_gemm<T, OutT, true>(A, B, C, M, N, K, lda, ldb, ldc, s, bias, resid, ldr)
                 : dispatch_gemm<T, OutT, false>(A, B, C, M, N, K, lda, ldb, ldc, s, bias, resid, ldr);
}

template <int WM, int WN>
int launch_w8a16(const f16* A, const int8_t* W, const f16* scales, f16* C, int64_t M, int64_t N, int64_t K,
                 hipStream_t s) {
  constexpr int BM = 2 * WM * 32, BN = 2 * WN * 32;
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  if (K % BK2 == 0 && K < (1 << 21)) {
    constexpr int NS = WM <= 2 ? 4 : 2;
    if ((K / BK2) % NS == 0)
      hipLaunchKernelGGL((gemm_kernel_k64<f16, f16, WM, WN, true, false, true, NS>), dim3(tiles_m * tiles_n),
                         dim3(256), 0, s, A, static_cast<const void*>(W), C, (int)M, (int)N, (int)K, K, K, N, tiles_m,
                         tiles_n, scales);
    else
      hipLaunchKernelGGL((gemm_kernel_k64<f16, f16, WM, WN, true, true, true, NS>), dim3(tiles_m * tiles_n),
                         dim3(256), 0, s, A, static_cast<const void*>(W), C, (int)M, (int)N, (int)K, K, K, N, tiles_m,
                         tiles_n, scales);
    return launch_status();
  }
  if ((K / BK) % 4 == 0)
    hipLaunchKernelGGL((gemm_kernel<f16, f16, WM, WN, true, false, true>), dim3(tiles_m * tiles_n), dim3(256), 0, s, A,
                       static_cast<const void*>(W), C, (int)M, (int)N, (int)K, K, K, N, tiles_m, tiles_n, scales);
  else
    hipLaunchKernelGGL((gemm_kernel<f16, f16, WM, WN, true, true, true>), dim3(tiles_m * tiles_n), dim3(256), 0, s, A,
                       static_cast<const void*>(W), C, (int)M, (int)N, (int)K, K, K, N, tiles_m, tiles_n, scales);
  return launch_status();
}

// one thread per element: only ever used for the result of a product over an empty inner dimension
__global__ __launch_bounds__(256)
void fill_zero_kernel(char* __restrict__ C, int64_t rows, int64_t cols, int64_t ld, int elem_size) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * cols) return;
  char* p = C + ((i / cols) * ld + i % cols) * elem_size;
  for (int b = 0; b < elem_size; ++b) p[b] = 0;
}

}  // namespace

int fill_zero_2d(void* C, int64_t rows, int64_t cols, int64_t ld, int elem_size, hipStream_t stream) {
  const int64_t blocks = (rows * cols + 255) / 256;
  if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, static_cast<char*>(C), rows, cols,
                     ld, elem_size);
  return launch_status();
}

// Any K and alignment: the register-staged 128x128 kernel with int8 B (zero points and a per-tensor scale included).
int gemm_w8a16_any_shape(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales,
                         const int8_t* zero_points, int per_tensor, f16* C, hipStream_t stream) {
  const int64_t tiles_m = (M + 127) / 128, tiles_n = (N + 127) / 128;
  if (tiles_m * tiles_n > 0x7fffffff || K > 0x7fffffff - 64) return HEXMI_ENOTSUP;
  hipLaunchKernelGGL((gemm_kernel_any<f16, f16, true, true>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, stream, A,
                     static_cast<const void*>(W), C, (int)M, (int)N, (int)K, K, K, N, (int)tiles_m, (int)tiles_n, nullptr,
                     nullptr, 0, scales, zero_points, per_tensor);
  return launch_status();
}

// K % 32 == 0, N % 8 == 0, 16-byte aligned A / W / C / scales (checked by the caller).
int gemm_w8a16_tiled(int64_t M, int64_t N, int64_t K, const f16* A, const int8_t* W, const f16* scales, f16* C,
                     hipStream_t stream) {
  if (prefer_large_tiles(M, N)) return launch_w8a16<4, 4>(A, W, scales, C, M, N, K, stream);
  return launch_w8a16<2, 2>(A, W, scales, C, M, N, K, stream);
}

}  // namespace hexmi

using namespace hexmi;

extern "C" int hexmi_gemm_ex(int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb,
                             void* C, int64_t ldc, const void* bias, const void* residual, int64_t ldr, int in_dtype,
                             int out_dtype, int trans_b, hexmi_stream_t stream) {
  if (M < 0 || N < 0 || K < 0) return HEXMI_EINVAL;
  if (M == 0 || N == 0) return HEXMI_OK;
  if (!C || (K > 0 && (!A || !B))) return HEXMI_EINVAL;
  if (lda < K || ldc < N || ldb < (trans_b ? K : N) || (residual && ldr < N)) return HEXMI_EINVAL;
  if (M > 0x7fffffff || N > 0x7fffffff || K > 0x7fffffff) return HEXMI_ENOTSUP;
  hipStream_t s = as_stream(stream);
  begin_call();
  if (K == 0 && !bias && !residual) {                        // an empty sum: C = 0, as torch.matmul gives
    const int esz = dtype_size(out_dtype);
    const bool known = (in_dtype == HEXMI_F32 && out_dtype == HEXMI_F32) ||
                       ((in_dtype == HEXMI_F16 || in_dtype == HEXMI_BF16) && (out_dtype == in_dtype || out_dtype == HEXMI_F32));
    return known ? fill_zero_2d(C, M, N, ldc, esz, s) : HEXMI_ENOTSUP;
  }
  if (K == 0) return HEXMI_ENOTSUP;                          // bias / residual of an empty product: not provided
  const bool tb = trans_b != 0;
  if (in_dtype == HEXMI_F32 && out_dtype == HEXMI_F32) return launch_f32(tb, A, B, C, M, N, K, lda, ldb, ldc, s, bias, residual, ldr);
  if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F16) return dispatch_trans<f16, f16>(tb, A, B, C, M, N, K, lda, ldb, ldc, s, bias, residual, ldr);
  if (in_dtype == HEXMI_F16 && out_dtype == HEXMI_F32) return dispatch_trans<f16, float>(tb, A, B, C, M, N, K, lda, ldb, ldc, s, bias, residual, ldr);
  if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_BF16) return dispatch_trans<bf16, bf16>(tb, A, B, C, M, N, K, lda, ldb, ldc, s, bias, residual, ldr);
  if (in_dtype == HEXMI_BF16 && out_dtype == HEXMI_F32) return dispatch_trans<bf16, float>(tb, A, B, C, M, N, K, lda, ldb, ldc, s, bias, residual, ldr);
  return HEXMI_ENOTSUP;
}

extern "C" int hexmi_gemm(int64_t M, int64_t N, int64_t K, const void* A, int64_t lda, const void* B, int64_t ldb,
                          void* C, int64_t ldc, int in_dtype, int out_dtype, int trans_b, hexmi_stream_t stream) {
  return hexmi_gemm_ex(M, N, K, A, lda, B, ldb, C, ldc, nullptr, nullptr, 0, in_dtype, out_dtype, trans_b, stream);
}

extern "C" int hexmi_matmul_f16f16_f32(int64_t n_row, int64_t n_col, int64_t n_inner, float* out, const void* act,
                                       const void* w, hexmi_stream_t stream) {
  return hexmi_gemm(n_row, n_col, n_inner, act, n_inner, w, n_col, out, n_col, HEXMI_F16, HEXMI_F32, 0, stream);
}
