// Row reductions: softmax, RMSNorm, LayerNorm. Single pass over HBM: a row is loaded once with 16-byte
// non-temporal accesses, kept in registers as fp32, reduced with wavefront butterflies (plus one LDS exchange per
// reduction when a row spans several waves), and stored once.
//
//   rows up to 4 KiB  : one 64-lane wave per row, four rows per workgroup, no LDS, no barrier
//   rows up to 128 KiB: 256 .. 1024 threads per row with two to eight 16-byte chunks per thread (more, shorter
//                       waves keep more of HBM busy than one long wave per row)
//   anything else (or misaligned): generic strided kernel, row re-read from L2
#include "hexmi_common.h"
#include <type_traits>

namespace hexmi {
namespace {

template <typename T> struct Vec16 {               // one 16-byte global access
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p) {
  Vec16<T> r;
  *reinterpret_cast<u32x4*>(r.v) = *reinterpret_cast<const u32x4*>(p);
  return r;
}
template <typename T>
__device__ __forceinline__ void store16(T* p, const Vec16<T>& r) {
  *reinterpret_cast<u32x4*>(p) = *reinterpret_cast<const u32x4*>(r.v);
}
// Streaming variants: the row is touched exactly once, so keep it out of the
// way of resident data (weights, bias) in L2.
template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T* p) {
  Vec16<T> r;
  *reinterpret_cast<u32x4*>(r.v) = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return r;
}
template <typename T>
__device__ __forceinline__ void store16_stream(T* p, const Vec16<T>& r) {
  __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(r.v), reinterpret_cast<u32x4*>(p));
}

// Rows that do not start on 16-byte boundaries or do not end on a chunk boundary (RAGGED tiles): a whole chunk is one
// 16-byte access at the alignment of the element type, which the hardware takes; the row's last, partial chunk goes
// element by element (n of them; the rest of a loaded chunk is zero bits).
template <typename T>
__device__ __forceinline__ Vec16<T> load16_any(const T* p, int n) {
  Vec16<T> r;
  if (n >= Vec16<T>::N) {
    __builtin_memcpy(r.v, p, 16);
  } else {
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i) r.v[i] = i < n ? p[i] : T(0.0f);
  }
  return r;
}
template <typename T>
__device__ __forceinline__ void store16_any(T* p, const Vec16<T>& r, int n) {
  if (n >= Vec16<T>::N) {
    __builtin_memcpy(p, r.v, 16);
  } else {
#pragma unroll
    for (int i = 0; i < Vec16<T>::N; ++i)
      if (i < n) p[i] = r.v[i];
  }
}

// Reduce across the WAVES waves that share a row through LDS. `red` holds one float per wave and must not be
// reused by another reduction of the same kernel (each reduction gets its own slots, so one barrier suffices);
// every thread returns the combined value.
template <bool IS_MAX, int WAVES>
__device__ __forceinline__ float block_reduce(float v, float* red, int wave_in_row) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if constexpr (WAVES == 1) return v;
  if (threadIdx.x % kWave == 0) red[wave_in_row] = v;
  __syncthreads();
  float r = red[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) r = IS_MAX ? fmaxf(r, red[w]) : r + red[w];
  return r;
}

enum RowOp { kSoftmax = 0, kRmsNorm = 1, kLayerNorm = 2 };

// The same 16 bytes as a value the compiler has not seen before (no instruction). A conversion of it is then a
// conversion of its own, in the block that uses it, where it can fold into the arithmetic; without this the
// conversions of a row's two or three passes are merged into one, done once and kept as sixteen floats.
template <typename T>
__device__ __forceinline__ void fresh(Vec16<T>& r) {
  u32x4 bits = *reinterpret_cast<const u32x4*>(r.v);
  asm volatile("" : "+v"(bits));
  *reinterpret_cast<u32x4*>(r.v) = bits;
}

// 1 / sqrt(x) for x well inside the normal range (a variance plus eps): the hardware estimate (v_rsq_f32, about one
// ulp) and one Newton step, five instructions. The correctly rounded square root followed by the correctly rounded
// division, which every thread of a row would execute, is forty: a fifth of all the vector instructions of a
// LayerNorm row group. The result is within an ulp of theirs.
// 1 / x the same way (v_rcp_f32 and one Newton step, three instructions for the correctly rounded division's ten),
// for the sum of a softmax row: 1 <= x <= the row length.
__device__ __forceinline__ float rcp_newton(float x) {
  const float y = __builtin_amdgcn_rcpf(x);
  return fmaf(fmaf(-x, y, 1.0f), y, y);
}
// Outside that range the estimate itself is the answer (x = 0: inf, x = inf: 0, NaN: NaN) and the step, which would
// multiply 0 by inf, is skipped.
__device__ __forceinline__ float rsqrt_newton(float x) {
  const float y = __builtin_amdgcn_rsqf(x);
  const float e = fmaf(-(x * y), y, 1.0f);              // 1 - x y^2
  const float r = fmaf(0.5f * y, e, y);
  return (y > 0.0f && y < INFINITY) ? r : y;
}

// THREADS threads cooperate on one row (THREADS == 64: a wave per row, several
// rows per workgroup). Each thread owns CHUNKS 16-byte chunks, chunk c of
// thread t covering elements [(c*THREADS + t)*N, +N).
//
// PIPE (large problems whose shape fills the tile exactly: cols == CHUNKS * THREADS * N and
// rows % ROWS_PER_BLOCK == 0, so no access is masked): the grid is a few workgroups per CU and each walks row
// groups blockIdx.x, +gridDim.x, ...; the loads of the next group are issued before the current one is reduced,
// so every wave always has a row in flight and HBM sees a steady stream instead of load / reduce / store phases.
// Weight and bias stay in registers for the walk. The stores of a group are unconditional, so the wait for the
// prefetched loads that follows them can leave exactly those stores outstanding; a store under a condition would
// turn that wait into a wait for everything, write acknowledgements included. For the same reason LayerNorm's
// per-row mean / rstd (one lane stores them) are written one group late, between the wait for the loads and the
// issue of the next ones.
// Without PIPE a workgroup handles exactly one row group (gridDim.x == number of groups) and accesses are masked.
// RAGGED (never with PIPE): rows at any alignment and of any length; the masks are per element.
// SPAN (softmax, RAGGED, x and y rows equally far off a 16-byte boundary): the row is walked as the aligned 16-byte
// chunks that cover it, the first of them starting up to N - 1 elements before the row. Whole chunks are read and
// written aligned (the bytes of the first and last chunk outside the row are read, sit inside the same 16 aligned
// bytes as the row's own, and are masked); only the row's two end chunks are stored element by element. An access
// at the alignment of the element type costs about 1.6 times an aligned one.
template <typename T, int OP, int CHUNKS, int THREADS, int ROWS_PER_BLOCK, bool PIPE, bool RAGGED = false, bool SPAN = false>
__global__ __launch_bounds__(THREADS * ROWS_PER_BLOCK)
void row_kernel(const T* __restrict__ x, T* __restrict__ y, const T* __restrict__ w,
                const T* __restrict__ b, float* __restrict__ mean_out, float* __restrict__ rstd_out,
                int64_t rows, int cols, int64_t ld_x, int64_t ld_y, float eps) {
  constexpr bool FULL = PIPE;
  static_assert(!(PIPE && RAGGED), "the pipelined walk is for exact tiles");
  static_assert(!SPAN || (RAGGED && OP == kSoftmax), "aligned spans: softmax over ragged rows");
  // MIX (fp16 norms, pipelined walk): the row is kept as loaded and every first use converts it inside the
  // arithmetic (v_fma_mix_f32 reads an fp16 half of a register as one operand of an fp32 fma, at the issue cost of
  // a plain fma), instead of sixteen conversions per thread and row up front. The norms issue vector instructions
  // a third to a half of the time, and a sixth fewer of them is +1.3 % for RMSNorm and +0.6 % for LayerNorm (six
  // alternating runs on one box). The loaded row lives until the end of the group in registers of its own, copied
  // from the load buffer before the next group's loads are issued into it. (Two load buffers that the walk
  // alternates between, which saves those copies, measured 2 % SLOWER than no change at all.)
  constexpr bool MIX = PIPE && OP != kSoftmax && std::is_same<T, f16>::value;
  constexpr int N = Vec16<T>::N;
  constexpr int WAVES = THREADS / kWave;
  constexpr int SLOTS = PIPE ? 2 : 1;                // consecutive groups alternate slots: a fast wave may start
                                                     // the next group while a slow one still reads this one's sums
  __shared__ float red_a[SLOTS][ROWS_PER_BLOCK][WAVES];     // first reduction (max / mean)
  __shared__ float red_b[SLOTS][ROWS_PER_BLOCK][WAVES];     // second reduction (sum / variance)
  const int t = threadIdx.x % THREADS;
  const int row_in_block = threadIdx.x / THREADS;
  const int wave_in_row = t / kWave;
  const int64_t groups = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  const float inv_n = 1.0f / (float)cols;

  Vec16<T> wv[CHUNKS], bv[CHUNKS];
  float wf[PIPE ? CHUNKS : 1][N], bf[PIPE ? CHUNKS : 1][N];   // PIPE: weight and bias resident as fp32
  if constexpr (PIPE && OP != kSoftmax) {
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int col = (c * THREADS + t) * N;
      if (w) wv[c] = load16(w + col);
      if (OP == kLayerNorm && b) bv[c] = load16(b + col);
#pragma unroll
      for (int i = 0; i < N; ++i) {
        wf[c][i] = w ? to_f32<T>(wv[c].v[i]) : 1.0f;
        bf[c][i] = (OP == kLayerNorm && b) ? to_f32<T>(bv[c].v[i]) : 0.0f;
      }
    }
  }

  // Rows past the end (last group only) are computed on the last row and not stored, so every wave reaches the
  // barriers.
  auto row_of = [&](int64_t g) {
    const int64_t r = g * ROWS_PER_BLOCK + row_in_block;
    return r < rows ? r : rows - 1;
  };
  // Chunks past the end of the row load column 0 instead (and are ignored): the loads stay free of branches,
  // which lets them be issued back to back and waited for only where their values are used.
  // SPAN: elements between the 16-byte boundary at or below the row's first element and that element; positions
  // count from the boundary, the row is positions lead .. lead + cols - 1
  int lead = 0;
  if constexpr (SPAN)
    lead = (int)((reinterpret_cast<uintptr_t>(x + row_of(blockIdx.x) * ld_x) / sizeof(T)) % N);
  const int span = cols + lead;
  int load_col[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) load_col[c] = (c * THREADS + t) * N < span ? (c * THREADS + t) * N : 0;
  // RAGGED: elements of chunk c inside the row (a chunk past the end stands in for column 0's, as above)
  auto left = [&](int c) { return cols - load_col[c]; };
  Vec16<T> raw_a[CHUNKS];
  {
    const T* xr = x + row_of(blockIdx.x) * ld_x - lead;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      if constexpr (RAGGED && !SPAN) raw_a[c] = load16_any(xr + load_col[c], left(c));
      else raw_a[c] = load16_stream(xr + load_col[c]);
    }
  }
  float one = 1.0f, zero = 0.0f;                       // opaque, so that x * one + y and x * y + zero stay fused
  if constexpr (MIX) asm volatile("" : "+v"(one), "+v"(zero));   // multiply-adds (the form that converts on the fly)

  int slot = 0;
  int64_t g = blockIdx.x;
  float stat_mean = 0.0f, stat_rstd = 0.0f;           // LayerNorm statistics of the previous group, not yet stored
  int64_t stat_row = -1;
  auto flush_stats = [&]() {
    if constexpr (OP == kLayerNorm) {
      if (t == 0 && stat_row >= 0) {
        if (mean_out) mean_out[stat_row] = stat_mean;
        if (rstd_out) rstd_out[stat_row] = stat_rstd;
      }
    }
  };
  // One row group; PREFETCH (a compile-time flag, so the walk below has no branch around the loads) issues the
  // loads of group g + gridDim.x before the reductions of group g.
  // raw_in: the group's row as loaded; next: where the loads of the following group go (the same buffer)
  auto process = [&](auto prefetch_tag, Vec16<T>* raw_in, Vec16<T>* next) {
    Vec16<T> raw[CHUNKS];                               // this group's row, live to the end of the group with MIX
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) raw[c] = raw_in[c];
    constexpr bool PREFETCH = decltype(prefetch_tag)::value;
    const int64_t row = g * ROWS_PER_BLOCK + row_in_block;
    const bool row_valid = FULL || row < rows;
    T* yr = y + (row_valid ? row : rows - 1) * ld_y;
    float v[CHUNKS][N];
    if constexpr (!MIX) {
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        const bool in = FULL || (c * THREADS + t) * N < span;
#pragma unroll
        for (int i = 0; i < N; ++i)
          v[c][i] = in && (!RAGGED || (c * THREADS + t) * N + i < span) && (!SPAN || (c * THREADS + t) * N + i >= lead)
                        ? to_f32<T>(raw[c].v[i])
                        : (OP == kSoftmax ? -INFINITY : 0.0f);
      }
    }
    flush_stats();
    if constexpr (PREFETCH) {
      const T* xn = x + row_of(g + gridDim.x) * ld_x;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) next[c] = load16_stream(xn + load_col[c]);
    }

    if constexpr (OP == kSoftmax) {
      float m = -INFINITY;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
        for (int i = 0; i < N; ++i) m = fmaxf(m, v[c][i]);
      m = block_reduce<true, WAVES>(m, red_a[slot][row_in_block], wave_in_row);
      float s = 0.0f;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
        for (int i = 0; i < N; ++i) { v[c][i] = __expf(v[c][i] - m); s += v[c][i]; }
      s = block_reduce<false, WAVES>(s, red_b[slot][row_in_block], wave_in_row);
      const float inv = rcp_newton(s);
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * THREADS + t) * N;
        if (FULL || (col < span && row_valid)) {
          Vec16<T> o;
#pragma unroll
          for (int i = 0; i < N; ++i) o.v[i] = from_f32<T>(v[c][i] * inv);
          if constexpr (SPAN) {
            T* ya = yr - lead + col;                      // 16-byte aligned: y's rows are as far off as x's
            if (col >= lead && col + N <= span) {
              store16_stream(ya, o);
            } else {
#pragma unroll
              for (int i = 0; i < N; ++i)
                if (col + i >= lead && col + i < span) ya[i] = o.v[i];
            }
          } else if constexpr (RAGGED) {
            store16_any(yr + col, o, cols - col);
          } else {
            store16_stream(yr + col, o);
          }
        }
      }
    } else {
      float mean = 0.0f;
      if constexpr (OP == kLayerNorm) {
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
          for (int i = 0; i < N; ++i) {
            if constexpr (MIX) s = fmaf(to_f32<T>(raw[c].v[i]), one, s);
            else s += v[c][i];                          // masked slots hold 0
          }
        mean = block_reduce<false, WAVES>(s, red_a[slot][row_in_block], wave_in_row) * inv_n;
      }
      float q = 0.0f;
      if constexpr (MIX && OP == kLayerNorm) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) fresh(raw[c]);
      }
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        if (FULL || (c * THREADS + t) * N < cols) {
#pragma unroll
          for (int i = 0; i < N; ++i) {
            if constexpr (MIX && OP == kLayerNorm) {
              v[c][i] = fmaf(to_f32<T>(raw[c].v[i]), one, -mean);
              q = fmaf(v[c][i], v[c][i], q);
            } else if constexpr (MIX) {
              q = fmaf(to_f32<T>(raw[c].v[i]), to_f32<T>(raw[c].v[i]), q);
            } else if (!RAGGED || (c * THREADS + t) * N + i < cols) {
              v[c][i] -= mean;
              q += v[c][i] * v[c][i];
            }
          }
        }
      }
      q = block_reduce<false, WAVES>(q, red_b[slot][row_in_block], wave_in_row);
      if constexpr (MIX && OP == kRmsNorm) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) fresh(raw[c]);
      }
      const float rstd = rsqrt_newton(q * inv_n + eps);
      if constexpr (OP == kLayerNorm) {
        stat_mean = mean;
        stat_rstd = rstd;
        stat_row = row_valid ? row : -1;
      }
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * THREADS + t) * N;
        if (FULL || (col < cols && row_valid)) {
          Vec16<T> o;
          if constexpr (PIPE) {
            // (x - mean) * rstd * w + b with the last two steps fused; w = 1 / b = 0 stand in for absent operands
            if (OP == kLayerNorm && b) {
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] = fmaf(v[c][i] * rstd, wf[c][i], bf[c][i]);
            } else if constexpr (MIX && OP == kRmsNorm) {
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] = fmaf(to_f32<T>(raw[c].v[i]), rstd, zero) * wf[c][i];
            } else {
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] = v[c][i] * rstd * wf[c][i];
            }
          } else {
            if (w) {
              if constexpr (RAGGED) wv[c] = load16_any(w + col, cols - col);
              else wv[c] = load16(w + col);
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] = v[c][i] * rstd * to_f32<T>(wv[c].v[i]);
            } else {
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] = v[c][i] * rstd;
            }
            if (OP == kLayerNorm && b) {
              if constexpr (RAGGED) bv[c] = load16_any(b + col, cols - col);
              else bv[c] = load16(b + col);
#pragma unroll
              for (int i = 0; i < N; ++i) v[c][i] += to_f32<T>(bv[c].v[i]);
            }
          }
#pragma unroll
          for (int i = 0; i < N; ++i) o.v[i] = from_f32<T>(v[c][i]);
          if constexpr (RAGGED) store16_any(yr + col, o, cols - col);
          else store16_stream(yr + col, o);
        }
      }
    }
  };
  if constexpr (PIPE) {
    for (; g + gridDim.x < groups; g += gridDim.x, slot ^= 1) process(std::true_type{}, raw_a, raw_a);
  }
  if (g < groups) process(std::false_type{}, raw_a, raw_a);
  flush_stats();
}

// Any shape / alignment: 256 threads per row, scalar accesses, the row is read
// again for each sweep (it stays in L2 for any row this path is chosen for).
template <typename T, int OP>
__global__ __launch_bounds__(256)
void row_kernel_generic(const T* __restrict__ x, T* __restrict__ y, const T* __restrict__ w,
                        const T* __restrict__ b, float* __restrict__ mean_out, float* __restrict__ rstd_out,
                        int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y, float eps) {
  constexpr int WAVES = 4;
  __shared__ float red_a[WAVES];
  __shared__ float red_b[WAVES];
  const int wave_in_row = threadIdx.x / kWave;
  const int64_t row = blockIdx.x;
  const T* xr = x + row * ld_x;
  T* yr = y + row * ld_y;
  const int t = threadIdx.x;
  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
    for (int64_t i = t; i < cols; i += 256) m = fmaxf(m, to_f32<T>(xr[i]));
    m = block_reduce<true, WAVES>(m, red_a, wave_in_row);
    float s = 0.0f;
    for (int64_t i = t; i < cols; i += 256) s += __expf(to_f32<T>(xr[i]) - m);
    s = block_reduce<false, WAVES>(s, red_b, wave_in_row);
    const float inv = 1.0f / s;
    for (int64_t i = t; i < cols; i += 256) yr[i] = from_f32<T>(__expf(to_f32<T>(xr[i]) - m) * inv);
  } else {
    const float inv_n = 1.0f / (float)cols;
    float mean = 0.0f;
    if constexpr (OP == kLayerNorm) {
      float s = 0.0f;
      for (int64_t i = t; i < cols; i += 256) s += to_f32<T>(xr[i]);
      mean = block_reduce<false, WAVES>(s, red_a, wave_in_row) * inv_n;
    }
    float q = 0.0f;
    for (int64_t i = t; i < cols; i += 256) { float d = to_f32<T>(xr[i]) - mean; q += d * d; }
    q = block_reduce<false, WAVES>(q, red_b, wave_in_row);
    const float rstd = 1.0f / sqrtf(q * inv_n + eps);
    if constexpr (OP == kLayerNorm) {
      if (t == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
      }
    }
    for (int64_t i = t; i < cols; i += 256) {
      float o = (to_f32<T>(xr[i]) - mean) * rstd;
      if (w) o *= to_f32<T>(w[i]);
      if (OP == kLayerNorm && b) o += to_f32<T>(b[i]);
      yr[i] = from_f32<T>(o);
    }
  }
}

// ---- rows split over several workgroups -------------------------------------------------------------------------
// A row that one workgroup cannot hold (more than 128 KiB), or a problem of so few rows that one workgroup per row
// leaves most CUs idle, is cut into parts of part_cols columns. Pass 1 reduces every part on its own, from
// registers, and leaves its statistics in a workspace; pass 2 merges the statistics of the row's parts, reads its
// part again (from L2 when the problem is small) and writes the result.
//   softmax: (m_p, l_p) = (max, sum exp(x - m_p)); merged as in the online form of
//            test/python/triton/test_online_softmax.py:60-71 (m = max(m_i, m_ij); l = l * exp(m_i - m) + l_ij), which is
//            associative: m = max_p m_p, l = sum_p l_p exp(m_p - m), summed in a fixed order.
//   RMSNorm: sum of squares. LayerNorm: (mean_p, M2_p = sum (x - mean_p)^2), merged to mean = sum n_p mean_p / n and
//            M2 = sum (M2_p + n_p (mean_p - mean)^2): the two-pass variance of the reference kernel
//            (test/python/triton/test_layer_norm.py:60-72) without a third sweep.
// A part is CHUNKS 16-byte chunks per thread of a 256-thread workgroup; chunks past the part or the row are masked.
constexpr int kPartThreads = 256;

template <typename T, int CHUNKS>
struct PartTile {
  static constexpr int N = Vec16<T>::N;
  float v[CHUNKS][N];
  bool in[CHUNKS];
  int col[CHUNKS];
  // loads part `part` of the row at xr; masked slots hold `fill`
  __device__ __forceinline__ void load(const T* xr, int64_t cols, int64_t part_cols, int64_t part, float fill) {
    const int64_t c0 = part * part_cols;
    const int64_t c1 = c0 + part_cols < cols ? c0 + part_cols : cols;
    Vec16<T> raw[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int64_t at = c0 + (int64_t)(c * kPartThreads + threadIdx.x) * N;
      in[c] = at < c1;
      col[c] = (int)(in[c] ? at - c0 : 0);
      raw[c] = load16(xr + c0 + col[c]);
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < N; ++i) v[c][i] = in[c] ? to_f32<T>(raw[c].v[i]) : fill;
  }
};

template <typename T, int OP, int CHUNKS>
__global__ __launch_bounds__(kPartThreads)
void part_stats_kernel(const T* __restrict__ x, float* __restrict__ stats, int64_t cols, int64_t ld_x,
                       int64_t part_cols, int64_t parts) {
  constexpr int N = Vec16<T>::N;
  constexpr int WAVES = kPartThreads / kWave;
  __shared__ float red_a[WAVES];
  __shared__ float red_b[WAVES];
  const int64_t row = blockIdx.x / parts, part = blockIdx.x % parts;
  const int wave = threadIdx.x / kWave;
  PartTile<T, CHUNKS> tile;
  tile.load(x + row * ld_x, cols, part_cols, part, OP == kSoftmax ? -INFINITY : 0.0f);
  float s0, s1 = 0.0f;
  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < N; ++i) m = fmaxf(m, tile.v[c][i]);
    m = block_reduce<true, WAVES>(m, red_a, wave);
    float l = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < N; ++i) l += __expf(tile.v[c][i] - m);     // masked slots: exp(-inf) = 0
    s0 = m;
    s1 = block_reduce<false, WAVES>(l, red_b, wave);
    if (m == -INFINITY) s1 = 0.0f;                   // a part of -inf only adds nothing (its own sum would be NaN)
  } else if constexpr (OP == kRmsNorm) {
    float q = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < N; ++i) q += tile.v[c][i] * tile.v[c][i];
    s0 = block_reduce<false, WAVES>(q, red_a, wave);
  } else {
    const int64_t c0 = part * part_cols;
    const float n_p = (float)(c0 + part_cols < cols ? part_cols : cols - c0);
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int i = 0; i < N; ++i) s += tile.v[c][i];
    const float mean = block_reduce<false, WAVES>(s, red_a, wave) / n_p;
    float q = 0.0f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
      if (tile.in[c]) {
#pragma unroll
        for (int i = 0; i < N; ++i) { const float d = tile.v[c][i] - mean; q += d * d; }
      }
    s0 = mean;
    s1 = block_reduce<false, WAVES>(q, red_b, wave);
  }
  if (threadIdx.x == 0) {
    stats[blockIdx.x * 2] = s0;
    stats[blockIdx.x * 2 + 1] = s1;
  }
}

template <typename T, int OP, int CHUNKS>
__global__ __launch_bounds__(kPartThreads)
void part_apply_kernel(const T* __restrict__ x, T* __restrict__ y, const T* __restrict__ w, const T* __restrict__ b,
                       float* __restrict__ mean_out, float* __restrict__ rstd_out, const float* __restrict__ stats,
                       int64_t cols, int64_t ld_x, int64_t ld_y, int64_t part_cols, int64_t parts, float eps) {
  constexpr int N = Vec16<T>::N;
  constexpr int WAVES = kPartThreads / kWave;
  __shared__ float red_a[WAVES];
  __shared__ float red_b[WAVES];
  const int64_t row = blockIdx.x / parts, part = blockIdx.x % parts;
  const int wave = threadIdx.x / kWave;
  const float* st = stats + row * parts * 2;
  // the row's own part first (its loads are in flight while the statistics are merged)
  PartTile<T, CHUNKS> tile;
  tile.load(x + row * ld_x, cols, part_cols, part, 0.0f);
  // merge: thread t takes parts t, t + 256, ... in order, then the threads are combined by the block reductions
  float a = 0.0f, scale = 0.0f;                    // softmax: a = max, scale = 1 / sum; norms: a = mean, scale = rstd
  if constexpr (OP == kSoftmax) {
    float m = -INFINITY;
    for (int64_t i = threadIdx.x; i < parts; i += kPartThreads) m = fmaxf(m, st[i * 2]);
    m = block_reduce<true, WAVES>(m, red_a, wave);
    float l = 0.0f;
    for (int64_t i = threadIdx.x; i < parts; i += kPartThreads) l += st[i * 2 + 1] * __expf(st[i * 2] - m);
    l = block_reduce<false, WAVES>(l, red_b, wave);
    a = m;
    scale = rcp_newton(l);
  } else if constexpr (OP == kRmsNorm) {
    float q = 0.0f;
    for (int64_t i = threadIdx.x; i < parts; i += kPartThreads) q += st[i * 2];
    q = block_reduce<false, WAVES>(q, red_a, wave);
    scale = rsqrt_newton(q / (float)cols + eps);
  } else {
    auto n_of = [&](int64_t i) { return (float)(i * part_cols + part_cols < cols ? part_cols : cols - i * part_cols); };
    float s = 0.0f;
    for (int64_t i = threadIdx.x; i < parts; i += kPartThreads) s += n_of(i) * st[i * 2];
    const float mean = block_reduce<false, WAVES>(s, red_a, wave) / (float)cols;
    float q = 0.0f;
    for (int64_t i = threadIdx.x; i < parts; i += kPartThreads) {
      const float d = st[i * 2] - mean;
      q += st[i * 2 + 1] + n_of(i) * d * d;
    }
    q = block_reduce<false, WAVES>(q, red_b, wave);
    a = mean;
    scale = rsqrt_newton(q / (float)cols + eps);
    if (part == 0 && threadIdx.x == 0) {
      if (mean_out) mean_out[row] = mean;
      if (rstd_out) rstd_out[row] = scale;
    }
  }
  const int64_t c0 = part * part_cols;
  T* yr = y + row * ld_y + c0;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    if (!tile.in[c]) continue;
    Vec16<T> o, wv, bv;
    if (OP != kSoftmax && w) wv = load16(w + c0 + tile.col[c]);
    if (OP == kLayerNorm && b) bv = load16(b + c0 + tile.col[c]);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float r;
      if constexpr (OP == kSoftmax) {
        r = __expf(tile.v[c][i] - a) * scale;
      } else {
        r = (tile.v[c][i] - a) * scale;
        if (w) r *= to_f32<T>(wv.v[i]);
        if (OP == kLayerNorm && b) r += to_f32<T>(bv.v[i]);
      }
      o.v[i] = from_f32<T>(r);
    }
    store16_stream(yr + tile.col[c], o);
  }
}

// The split of a (rows x cols) problem: part_cols == 0 means the single-pass kernels take it. block_cols > 0 asks for
// parts of that many columns (rounded up to whole 16-byte chunks, at most 32 KiB); block_cols == 0 leaves the choice
// to the library: rows of more than 128 KiB, and problems of fewer rows than half the CUs whose rows are at least
// 32 KiB, in parts of 4 .. 16 KiB so that there are about two workgroups per CU.
struct RowSplit {
  int64_t part_cols, parts;
  int chunks;
};
inline RowSplit plan_row_split(int64_t rows, int64_t cols, int64_t block_cols, int elem_size, int cus) {
  RowSplit r = {0, 0, 0};
  const int64_t n = 16 / elem_size;                // elements per 16-byte chunk
  const int64_t unit = kPartThreads * n;           // elements one chunk per thread covers
  const int64_t row_bytes = cols * elem_size;
  int64_t part = 0;
  if (block_cols > 0) {
    part = (block_cols + n - 1) / n * n;
    if (part > 8 * unit) part = 8 * unit;
    if (part >= cols) part = cols;                 // one part: still the two-pass form the caller asked for
  } else if (row_bytes > (128 << 10) || (rows * 2 < cus && row_bytes >= (32 << 10))) {
    int64_t bytes = cus > 0 ? row_bytes * rows / (2 * (int64_t)cus) : 0;
    bytes = bytes < 4096 ? 4096 : (bytes > 16384 ? 16384 : bytes);
    part = (bytes + 4095) / 4096 * 4096 / elem_size;
  } else {
    return r;
  }
  r.part_cols = part;
  r.parts = (cols + part - 1) / part;
  const int64_t per_thread = (part + unit - 1) / unit;
  r.chunks = per_thread <= 1 ? 1 : per_thread <= 2 ? 2 : per_thread <= 4 ? 4 : 8;
  if (rows * r.parts > 0x7fffffff) r = {0, 0, 0};
  return r;
}

template <typename T, int OP, int CHUNKS>
int launch_split(const RowSplit& sp, const T* x, T* y, const T* w, const T* b, float* mean, float* rstd, int64_t rows,
                 int64_t cols, int64_t ld_x, int64_t ld_y, float eps, float* stats, hipStream_t s) {
  const dim3 grid((unsigned)(rows * sp.parts));
  hipLaunchKernelGGL((part_stats_kernel<T, OP, CHUNKS>), grid, dim3(kPartThreads), 0, s, x, stats, cols, ld_x,
                     sp.part_cols, sp.parts);
  hipLaunchKernelGGL((part_apply_kernel<T, OP, CHUNKS>), grid, dim3(kPartThreads), 0, s, x, y, w, b, mean, rstd, stats,
                     cols, ld_x, ld_y, sp.part_cols, sp.parts, eps);
  return launch_status();
}

// Grid of a pipelined launch: about 32 KiB of loads in flight per CU (2048 / CHUNKS threads, each with CHUNKS
// 16-byte loads outstanding) measured fastest on MI355X: more resident workgroups shorten each one's walk and
// bring the load / reduce / store phases back, fewer leave HBM idle. A problem too small for every workgroup to
// walk at least four groups is launched with one group per workgroup instead.
constexpr int kPipeChunksPerCu = 2048;
constexpr int kPipeMinWalk = 4;

template <typename T, int OP, int CHUNKS, int THREADS, int RPB, bool PIPE>
int launch_grid(int64_t blocks, const T* x, T* y, const T* w, const T* b, float* mean, float* rstd, int64_t rows,
                int64_t cols, int64_t ld_x, int64_t ld_y, float eps, hipStream_t s) {
  hipLaunchKernelGGL((row_kernel<T, OP, CHUNKS, THREADS, RPB, PIPE>), dim3((unsigned)blocks), dim3(THREADS * RPB), 0,
                     s, x, y, w, b, mean, rstd, rows, (int)cols, ld_x, ld_y, eps);
  return launch_status();
}

// MAY_PIPE: whether the tile has a pipelined instantiation at all (the widest tiles do not: one workgroup of
// 1024 threads per CU leaves nothing to overlap with). threads_per_cu <= 0 selects the default.
template <typename T, int OP, int CHUNKS, int THREADS, int RPB, bool MAY_PIPE>
int launch_tile(const T* x, T* y, const T* w, const T* b, float* mean, float* rstd, int64_t rows,
                int64_t cols, int64_t ld_x, int64_t ld_y, float eps, hipStream_t s, int threads_per_cu = 0) {
  constexpr int N = 16 / sizeof(T);
  const int64_t groups = (rows + RPB - 1) / RPB;
  if constexpr (MAY_PIPE) {
    if (cols == (int64_t)CHUNKS * THREADS * N && rows % RPB == 0) {
      if (threads_per_cu <= 0) threads_per_cu = kPipeChunksPerCu / CHUNKS;
      const int per_cu = threads_per_cu / (THREADS * RPB) > 0 ? threads_per_cu / (THREADS * RPB) : 1;
      const int64_t resident = (int64_t)hexmi_num_cus() * per_cu;
      if (resident > 0 && groups >= kPipeMinWalk * resident)
        return launch_grid<T, OP, CHUNKS, THREADS, RPB, true>(resident, x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y,
                                                              eps, s);
    }
  }
  return launch_grid<T, OP, CHUNKS, THREADS, RPB, false>(groups, x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, s);
}

template <typename T, int OP>
int dispatch_rows(const void* xv, void* yv, const void* wv, const void* bv, float* mean, float* rstd,
                  int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y, float eps, hipStream_t s,
                  int64_t block_cols = 0, void* workspace = nullptr, int64_t workspace_bytes = 0) {
  const T* x = static_cast<const T*>(xv);
  T* y = static_cast<T*>(yv);
  const T* w = static_cast<const T*>(wv);
  const T* b = static_cast<const T*>(bv);
  constexpr int N = 16 / sizeof(T);
  const bool vec_ok = cols % N == 0 && ld_x % N == 0 && ld_y % N == 0 && aligned_to(x, 16) && aligned_to(y, 16) &&
                      (!w || aligned_to(w, 16)) && (!b || aligned_to(b, 16));
  if (vec_ok && workspace && aligned_to(workspace, 4)) {
    const RowSplit sp = plan_row_split(rows, cols, block_cols, (int)sizeof(T), hexmi_num_cus());
    if (sp.part_cols > 0) {
      if (workspace_bytes < rows * sp.parts * 8) return HEXMI_EINVAL;
      float* stats = static_cast<float*>(workspace);
#define HEXMI_SPLIT(C) return launch_split<T, OP, C>(sp, x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, stats, s)
      if (sp.chunks == 1) HEXMI_SPLIT(1);
      if (sp.chunks == 2) HEXMI_SPLIT(2);
      if (sp.chunks == 4) HEXMI_SPLIT(4);
      HEXMI_SPLIT(8);
#undef HEXMI_SPLIT
    }
  }
  const int64_t chunks = (cols + N - 1) / N;        // 16-byte chunks per row
  // softmax over many rows runs a little faster with half the usual loads in flight (one 256-thread workgroup per
  // CU at 1024 fp32 columns: 0.760 against 0.748 of the HBM figure at [65536,1024], A/B); the norms and small
  // problems do not
  const int tpc = (OP == kSoftmax && rows >= 16384) ? 1024 : 0;
#define HEXMI_TILE(C, TH, RPB, PIPE) \
  return launch_tile<T, OP, C, TH, RPB, PIPE>(x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, s, tpc / C)
  if (vec_ok && rows <= 0x7fffffff) {
    // about two to four 16-byte chunks per thread; rows narrower than 4 KiB stay inside one wave (no barrier)
    if (chunks <= 64 * 1) HEXMI_TILE(1, 64, 4, true);
    if (chunks <= 64 * 2) HEXMI_TILE(2, 64, 4, true);
    if (chunks <= 64 * 4) HEXMI_TILE(4, 64, 4, true);
    if (chunks <= 256 * 2) HEXMI_TILE(2, 256, 1, true);
    if (chunks <= 256 * 4) HEXMI_TILE(4, 256, 1, true);
    if (chunks <= 512 * 4) HEXMI_TILE(4, 512, 1, true);
    if (chunks <= 1024 * 4) HEXMI_TILE(4, 1024, 1, false);
    if (chunks <= 1024 * 8) HEXMI_TILE(8, 1024, 1, false);
  }
#undef HEXMI_TILE
  // Rows that are not whole aligned chunks (an odd number of columns, a view that starts anywhere): the same tiles
  // with per-element masks and accesses at the alignment of the element type; one pass over the row instead of the
  // three sweeps of the kernel below ([8192, 4097] fp16: softmax 62 us on that one, 24 us at 4096 columns).
#define HEXMI_RAGGED(C, TH, RPB) \
  { hipLaunchKernelGGL((row_kernel<T, OP, C, TH, RPB, false, true>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(TH * RPB), 0, s, \
                       x, y, w, b, mean, rstd, rows, (int)cols, ld_x, ld_y, eps); return launch_status(); }
  // softmax with x and y rows equally far off a 16-byte boundary (contiguous tensors with an odd number of columns,
  // equal column slices of aligned ones): aligned chunks over the span that covers the row, one chunk more at most
  if constexpr (OP == kSoftmax) {
    const bool same_offset = aligned_to(x, sizeof(T)) && aligned_to(y, sizeof(T)) &&
                             (reinterpret_cast<uintptr_t>(x) - reinterpret_cast<uintptr_t>(y)) % 16 == 0 &&
                             ((ld_x - ld_y) * (int64_t)sizeof(T)) % 16 == 0;
    const int64_t span_chunks = (cols + 2 * N - 2) / N;
    if (!vec_ok && same_offset && rows <= 0x7fffffff && cols < 0x7ffffff0) {
#define HEXMI_SPAN(C, TH, RPB) \
  { hipLaunchKernelGGL((row_kernel<T, OP, C, TH, RPB, false, true, true>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(TH * RPB), 0, \
                       s, x, y, w, b, mean, rstd, rows, (int)cols, ld_x, ld_y, eps); return launch_status(); }
      if (span_chunks <= 64 * 1) HEXMI_SPAN(1, 64, 4);
      if (span_chunks <= 64 * 2) HEXMI_SPAN(2, 64, 4);
      if (span_chunks <= 64 * 4) HEXMI_SPAN(4, 64, 4);
      if (span_chunks <= 256 * 2) HEXMI_SPAN(2, 256, 1);
      if (span_chunks <= 256 * 4) HEXMI_SPAN(4, 256, 1);
      if (span_chunks <= 512 * 4) HEXMI_SPAN(4, 512, 1);
      if (span_chunks <= 1024 * 4) HEXMI_SPAN(4, 1024, 1);
      if (span_chunks <= 1024 * 8) HEXMI_SPAN(8, 1024, 1);
#undef HEXMI_SPAN
    }
  }
  if (!vec_ok && rows <= 0x7fffffff) {
    if (chunks <= 64 * 1) HEXMI_RAGGED(1, 64, 4);
    if (chunks <= 64 * 2) HEXMI_RAGGED(2, 64, 4);
    if (chunks <= 64 * 4) HEXMI_RAGGED(4, 64, 4);
    if (chunks <= 256 * 2) HEXMI_RAGGED(2, 256, 1);
    if (chunks <= 256 * 4) HEXMI_RAGGED(4, 256, 1);
    if (chunks <= 512 * 4) HEXMI_RAGGED(4, 512, 1);
    if (chunks <= 1024 * 4) HEXMI_RAGGED(4, 1024, 1);
    if (chunks <= 1024 * 8) HEXMI_RAGGED(8, 1024, 1);
  }
#undef HEXMI_RAGGED
  if (rows > 0x7fffffff) return HEXMI_ENOTSUP;
  hipLaunchKernelGGL((row_kernel_generic<T, OP>), dim3((unsigned)rows), dim3(256), 0, s, x, y, w, b, mean, rstd, rows,
                     cols, ld_x, ld_y, eps);
  return launch_status();
}

template <int OP>
int dispatch_dtype(int dtype, const void* x, void* y, const void* w, const void* b, float* mean, float* rstd,
                   int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y, float eps, hipStream_t s,
                   int64_t block_cols = 0, void* ws = nullptr, int64_t ws_bytes = 0) {
  switch (dtype) {
    case HEXMI_F32: return dispatch_rows<float, OP>(x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, s, block_cols, ws, ws_bytes);
    case HEXMI_F16: return dispatch_rows<f16, OP>(x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, s, block_cols, ws, ws_bytes);
    case HEXMI_BF16: return dispatch_rows<bf16, OP>(x, y, w, b, mean, rstd, rows, cols, ld_x, ld_y, eps, s, block_cols, ws, ws_bytes);
    default: return HEXMI_ENOTSUP;
  }
}

}  // namespace
}  // namespace hexmi

using namespace hexmi;

extern "C" int hexmi_softmax(const void* x, void* y, int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y,
                             int dtype, hexmi_stream_t stream) {
  if (rows < 0 || cols < 0 || ld_x < cols || ld_y < cols) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kSoftmax>(dtype, x, y, nullptr, nullptr, nullptr, nullptr, rows, cols, ld_x, ld_y, 0.0f,
                                  as_stream(stream));
}

extern "C" int hexmi_rms_norm(const void* x, const void* weight, void* y, int64_t rows, int64_t cols, float eps,
                              int dtype, hexmi_stream_t stream) {
  if (rows < 0 || cols < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kRmsNorm>(dtype, x, y, weight, nullptr, nullptr, nullptr, rows, cols, cols, cols, eps,
                                  as_stream(stream));
}

extern "C" int hexmi_layer_norm(const void* x, const void* weight, const void* bias, void* y, float* mean,
                                float* rstd, int64_t rows, int64_t cols, float eps, int dtype,
                                hexmi_stream_t stream) {
  if (rows < 0 || cols < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kLayerNorm>(dtype, x, y, weight, bias, mean, rstd, rows, cols, cols, cols, eps,
                                    as_stream(stream));
}

// ---- the same operators with leading dimensions, a column-block size and a workspace ------------------------------

extern "C" int64_t hexmi_row_workspace(int64_t rows, int64_t cols, int64_t block_cols, int dtype) {
  const int esz = dtype_size(dtype);
  if (rows <= 0 || cols <= 0 || block_cols < 0 || esz < 2) return 0;
  const RowSplit sp = plan_row_split(rows, cols, block_cols, esz, hexmi_num_cus());
  return sp.part_cols > 0 ? rows * sp.parts * 8 : 0;
}

extern "C" int hexmi_softmax_ws(const void* x, void* y, int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y,
                                int64_t block_cols, int dtype, void* workspace, int64_t workspace_bytes,
                                hexmi_stream_t stream) {
  if (rows < 0 || cols < 0 || ld_x < cols || ld_y < cols || block_cols < 0 || workspace_bytes < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kSoftmax>(dtype, x, y, nullptr, nullptr, nullptr, nullptr, rows, cols, ld_x, ld_y, 0.0f,
                                  as_stream(stream), block_cols, workspace, workspace_bytes);
}

extern "C" int hexmi_rms_norm_ws(const void* x, const void* weight, void* y, int64_t rows, int64_t cols, int64_t ld_x,
                                 int64_t ld_y, float eps, int64_t block_cols, int dtype, void* workspace,
                                 int64_t workspace_bytes, hexmi_stream_t stream) {
  if (rows < 0 || cols < 0 || ld_x < cols || ld_y < cols || block_cols < 0 || workspace_bytes < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kRmsNorm>(dtype, x, y, weight, nullptr, nullptr, nullptr, rows, cols, ld_x, ld_y, eps,
                                  as_stream(stream), block_cols, workspace, workspace_bytes);
}

extern "C" int hexmi_layer_norm_ws(const void* x, const void* weight, const void* bias, void* y, float* mean,
                                   float* rstd, int64_t rows, int64_t cols, int64_t ld_x, int64_t ld_y, float eps,
                                   int64_t block_cols, int dtype, void* workspace, int64_t workspace_bytes,
                                   hexmi_stream_t stream) {
  if (rows < 0 || cols < 0 || ld_x < cols || ld_y < cols || block_cols < 0 || workspace_bytes < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  begin_call();
  return dispatch_dtype<kLayerNorm>(dtype, x, y, weight, bias, mean, rstd, rows, cols, ld_x, ld_y, eps,
                                    as_stream(stream), block_cols, workspace, workspace_bytes);
}
