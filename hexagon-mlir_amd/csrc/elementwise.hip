// Element-wise operators, block sums and rotary embedding: the small tutorial kernels of the reference
// (GELU-tanh, SiLU, rsqrt / sin / cos / exp, vector add / sub / mul / div, sum reduction, RoPE). All are one pass
// over HBM with 16-byte non-temporal accesses, four chunks in flight per thread, fp32 arithmetic.
#include "hexmi_common.h"

namespace hexmi {
namespace {

template <typename T> struct Chunk {                // one 16-byte global access
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};
template <typename T>
__device__ __forceinline__ Chunk<T> load_chunk(const T* p) {
  Chunk<T> r;
  *reinterpret_cast<u32x4*>(r.v) = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return r;
}
template <typename T>
__device__ __forceinline__ void store_chunk(T* p, const Chunk<T>& r) {
  __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(r.v), reinterpret_cast<u32x4*>(p));
}

// ---- unary ---------------------------------------------------------------------------------------------------
template <int OP>
__device__ __forceinline__ float unary(float x) {
  if constexpr (OP == HEXMI_GELU_TANH) {
    // 0.5*x*(1 + tanh(u)), u = 0.797885*x + 0.035677*x^3, tanh(u) = (1 - e^-2u) / (1 + e^-2u)
    // (test/python/triton/test_gelu.py:26-30,54). 0.5*(1 + tanh(u)) = 1 / (1 + e^-2u): the same function without
    // the cancellation in 1 + tanh(u) for negative u, and e^-2u = inf gives 0 instead of inf/inf.
    // v_exp_f32 and v_rcp_f32 (1 ulp each) and the constants folded into the exp2 argument,
    // e^-2u = 2^(x * (a + b x^2)), a = -2 log2(e) * 0.797885, b = -2 log2(e) * 0.035677, keep the kernel bound
    // by HBM rather than by the vector ALUs (eight fp16 elements per 16-byte access).
    constexpr float a = -2.0f * 1.44269504088896340736f * 0.797885f;
    constexpr float b = -2.0f * 1.44269504088896340736f * 0.035677f;
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * fmaf(b, x * x, a)));
  } else if constexpr (OP == HEXMI_SILU) {
    // x / (1 + e^-x), test/python/triton/test_silu.py:50
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
  } else if constexpr (OP == HEXMI_RSQRT) {
    return 1.0f / sqrtf(x);                          // test/python/triton/test_rsqrt.py:20-24
  } else if constexpr (OP == HEXMI_SIN) {
    return sinf(x);                                  // test/python/triton/test_math_ops.py:33-38
  } else if constexpr (OP == HEXMI_COS) {
    return cosf(x);                                  // test/python/triton/test_math_ops.py:25-30
  } else {
    return expf(x);
  }
}

constexpr int kEwThreads = 256;
// 16-byte chunks per thread (and loads in flight per thread). A/B on one box, GELU / SiLU fp16 [8192,4096]: two chunks
// 0.705 / 0.718 of the HBM figure, four 0.675 / 0.690, eight 0.686 / 0.715; 128-, 512- and 1024-thread workgroups
// were no better with either.
constexpr int kEwChunks = 2;
constexpr int kBinChunks = 2;                        // binary operators: chunks per operand and thread

template <typename T, int OP>
__global__ __launch_bounds__(kEwThreads)
void unary_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
  constexpr int N = Chunk<T>::N;
  const int64_t chunks = n / N;
  const int64_t c0 = (int64_t)blockIdx.x * (kEwThreads * kEwChunks) + threadIdx.x;
  Chunk<T> in[kEwChunks];
#pragma unroll
  for (int u = 0; u < kEwChunks; ++u) {
    const int64_t c = c0 + u * kEwThreads;
    in[u] = load_chunk(x + (c < chunks ? c : 0) * N);           // branch-free: out-of-range lanes re-read chunk 0
  }
#pragma unroll
  for (int u = 0; u < kEwChunks; ++u) {
    const int64_t c = c0 + u * kEwThreads;
    Chunk<T> out;
#pragma unroll
    for (int i = 0; i < N; ++i) out.v[i] = from_f32<T>(unary<OP>(to_f32<T>(in[u].v[i])));
    if (c < chunks) store_chunk(y + c * N, out);
  }
  if (blockIdx.x == 0 && threadIdx.x < n % N) {                  // the few elements past the last whole chunk
    const int64_t i = chunks * N + threadIdx.x;
    y[i] = from_f32<T>(unary<OP>(to_f32<T>(x[i])));
  }
}

// misaligned buffers: one element per thread
template <typename T, int OP>
__global__ __launch_bounds__(kEwThreads)
void unary_scalar_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (i < n) y[i] = from_f32<T>(unary<OP>(to_f32<T>(x[i])));
}

// ---- binary --------------------------------------------------------------------------------------------------
template <int OP>
__device__ __forceinline__ float binary(float a, float b) {
  if constexpr (OP == HEXMI_ADD) return a + b;       // test/python/triton/test_vec_add.py
  else if constexpr (OP == HEXMI_SUB) return a - b;
  else if constexpr (OP == HEXMI_MUL) return a * b;
  else return a / b;                                 // test/python/triton/test_vec_div_2d.py:52-55
}

template <typename T, int OP>
__global__ __launch_bounds__(kEwThreads)
void binary_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, int64_t n) {
  constexpr int N = Chunk<T>::N;
  constexpr int CH = kBinChunks;
  const int64_t chunks = n / N;
  const int64_t c0 = (int64_t)blockIdx.x * (kEwThreads * CH) + threadIdx.x;
  Chunk<T> ia[CH], ib[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const int64_t c = c0 + u * kEwThreads;
    ia[u] = load_chunk(a + (c < chunks ? c : 0) * N);
    ib[u] = load_chunk(b + (c < chunks ? c : 0) * N);
  }
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const int64_t c = c0 + u * kEwThreads;
    Chunk<T> out;
#pragma unroll
    for (int i = 0; i < N; ++i) out.v[i] = from_f32<T>(binary<OP>(to_f32<T>(ia[u].v[i]), to_f32<T>(ib[u].v[i])));
    if (c < chunks) store_chunk(y + c * N, out);
  }
  if (blockIdx.x == 0 && threadIdx.x < n % N) {
    const int64_t i = chunks * N + threadIdx.x;
    y[i] = from_f32<T>(binary<OP>(to_f32<T>(a[i]), to_f32<T>(b[i])));
  }
}

template <typename T, int OP>
__global__ __launch_bounds__(kEwThreads)
void binary_scalar_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * kEwThreads + threadIdx.x;
  if (i < n) y[i] = from_f32<T>(binary<OP>(to_f32<T>(a[i]), to_f32<T>(b[i])));
}

// ---- block sums ----------------------------------------------------------------------------------------------
// out[p] = sum(x[p*block .. (p+1)*block)), one workgroup per program of the reference's launch grid
// (test/python/triton/test_sum.py:30-36: `tl.store(output_ptr + pid, tl.sum(x))`). fp32 accumulation in a fixed
// order (per-thread strided partials, wave butterfly, waves in order): the result does not depend on timing.
// kSumThreads threads per program: 1024 for large blocks (a single program must pull its block through one CU),
// 256 for blocks up to 64 KiB (several 16-byte loads in flight per thread, a cheaper final exchange).
// TIn / TOut differ in the two-pass form below: fp32 partial sums of 16-bit inputs, a 16-bit result of fp32 partials.
template <typename T, typename TOut, int kSumThreads>
__global__ __launch_bounds__(kSumThreads)
void block_sum_kernel(const T* __restrict__ x, TOut* __restrict__ out, int64_t block, int64_t n) {
  constexpr int N = Chunk<T>::N;
  __shared__ float part[kSumThreads / kWave];
  const int64_t begin = (int64_t)blockIdx.x * block;
  const int64_t end = begin + block < n ? begin + block : n;
  const T* xb = x + begin;
  const int64_t len = end - begin;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const bool vec = reinterpret_cast<uintptr_t>(xb) % 16 == 0;
  const int64_t chunks = vec ? len / N : 0;
  int64_t c = threadIdx.x;
  for (; c + 3 * kSumThreads < chunks; c += 4 * kSumThreads) {   // four loads in flight
    Chunk<T> v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = load_chunk(xb + (c + u * kSumThreads) * N);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < N; ++i) acc[u] += to_f32<T>(v[u].v[i]);
  }
  for (; c < chunks; c += kSumThreads) {
    const Chunk<T> v = load_chunk(xb + c * N);
#pragma unroll
    for (int i = 0; i < N; ++i) acc[0] += to_f32<T>(v.v[i]);
  }
  for (int64_t i = chunks * N + threadIdx.x; i < len; i += kSumThreads) acc[1] += to_f32<T>(xb[i]);
  float s = wave_sum((acc[0] + acc[1]) + (acc[2] + acc[3]));
  if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < kSumThreads / kWave; ++w) t += part[w];
    out[blockIdx.x] = from_f32<TOut>(t);
  }
}

// A program is one workgroup (as it is one Triton program in the reference), so a launch of a few huge programs -
// the reference test sums 2^20 elements in ONE - would leave the chip idle. Programs of kTwoPassMinBlock elements
// and more are therefore summed in two passes when a scratch buffer is at hand: fp32 partial sums of runs of
// kSumRun elements by many workgroups (the runs of a program are whole when block % kSumRun == 0 or there is one
// program), then one sum per program over its partials. fp32 partials lose nothing for any input type.
// ---- rotary embedding ----------------------------------------------------------------------------------------
// x, y: [batch, seq, heads, feat] contiguous; features are rotated in adjacent pairs (2i, 2i+1) by the angle
// m * theta^(-2i/feat), m the sequence position (test/python/triton/test_rope.py:43-57 compute_thetas,
// :60-95 rope_reference_pytorch, :174-184 even / odd cases):
//   y[2i] = x[2i] cos - x[2i+1] sin,   y[2i+1] = x[2i] sin + x[2i+1] cos.
// A workgroup owns one sequence position; a thread owns one 16-byte chunk of the feature vector, computes the
// sines and cosines of its pairs once (in double: the angle m*freq is accurate to fp32 for any m) and walks all
// (batch, head) rows with them. The frequencies of a thread's pairs are a geometric sequence: one double-precision
// exp2 for the first, then a multiplication by pair_ratio = theta^(-2/feat) for each further pair (the set-up of a
// thread, four double exp2 and four sine / cosine pairs, was more vector work than its eight rows).
template <typename T>
__global__ __launch_bounds__(256)
void rope_kernel(const T* __restrict__ x, T* __restrict__ y, int batch, int seq, int heads, int feat, double log2_theta,
                 double pair_ratio) {
  constexpr int N = Chunk<T>::N;                     // elements per chunk (even)
  const int chunks = feat / N;                       // chunks per feature vector (feat % N == 0 on this path)
  const int rows_per_pass = 256 / chunks;            // (batch, head) rows handled side by side
  const int m = blockIdx.x;
  const int ch = threadIdx.x % chunks;
  const int r0 = threadIdx.x / chunks;
  if (r0 >= rows_per_pass) return;
  float cs[N / 2], sn[N / 2];
  // even feature index i2 = ch * N + 2 * p (the reference's `steps`): freq = theta^(-i2 / feat)
  double freq = exp2(-((double)(ch * N) / (double)feat) * log2_theta);
#pragma unroll
  for (int p = 0; p < N / 2; ++p) {
    if (p > 0) freq *= pair_ratio;
    // the angle m*freq in double, reduced in double to a quarter turn number q and a remainder in [-pi/4, pi/4]
    // (so it is accurate to fp32 for any m), then fp32 polynomials for the sine and cosine of the remainder (the
    // single-precision minimax coefficients of the Cephes library, errors near 1e-7) and the quadrant's swap and
    // signs: about half the instructions of sincosf, which reduces its argument once more
    double turns = (double)m * freq * 0.15915494309189533577;        // 1 / (2 pi)
    turns -= floor(turns);
    const double q = rint(turns * 4.0);                              // 0 .. 4
    const float rem = (float)((turns - 0.25 * q) * 6.28318530717958647692);
    const int qi = (int)q & 3;
    const float z = rem * rem;
    const float sp = fmaf(rem * z, fmaf(z, fmaf(z, -1.9515295891e-4f, 8.3321608736e-3f), -1.6666654611e-1f), rem);
    const float cp = fmaf(z * z, fmaf(z, fmaf(z, 2.443315711809948e-5f, -1.388731625493765e-3f), 4.166664568298827e-2f),
                          fmaf(z, -0.5f, 1.0f));
    float s = (qi & 1) ? cp : sp, c = (qi & 1) ? sp : cp;
    if (qi & 2) s = -s;
    if (qi == 1 || qi == 2) c = -c;
    cs[p] = c;
    sn[p] = s;
  }
  const int rows = batch * heads;                    // < 2^31: checked by the launcher
  // one row in flight per thread: with the next row's load issued ahead the kernel measured 5 % slower.
  // (batch, head) of the row advance with it: a division per row was a third of the loop's instructions
  const int step = rows_per_pass * (int)gridDim.y, step_b = step / heads, step_h = step % heads;
  int r = r0 + (int)blockIdx.y * rows_per_pass;
  int b = r / heads, h = r % heads;
  for (; r < rows; r += step, b += step_b, h += step_h) {
    if (h >= heads) {
      h -= heads;
      ++b;
    }
    const int64_t off = ((((int64_t)b * seq + m) * heads) + h) * feat + ch * N;
    const Chunk<T> in = load_chunk(x + off);
    Chunk<T> out;
#pragma unroll
    for (int p = 0; p < N / 2; ++p) {
      const float e = to_f32<T>(in.v[2 * p]), o = to_f32<T>(in.v[2 * p + 1]);
      out.v[2 * p] = from_f32<T>(e * cs[p] - o * sn[p]);
      out.v[2 * p + 1] = from_f32<T>(e * sn[p] + o * cs[p]);
    }
    store_chunk(y + off, out);
  }
}

// any feat (even), any alignment: one pair per thread
template <typename T>
__global__ __launch_bounds__(256)
void rope_pair_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t pairs_total, int seq, int heads, int feat,
                      double log2_theta) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= pairs_total) return;
  const int half = feat / 2;
  const int p = (int)(idx % half);
  const int64_t row = idx / half;                    // (b*seq + m)*heads + h
  const int m = (int)((row / heads) % seq);
  const double freq = exp2(-((double)(2 * p) / (double)feat) * log2_theta);
  double s, c;
  sincos((double)m * freq, &s, &c);
  const int64_t off = row * feat + 2 * p;
  const float e = to_f32<T>(x[off]), o = to_f32<T>(x[off + 1]);
  y[off] = from_f32<T>(e * (float)c - o * (float)s);
  y[off + 1] = from_f32<T>(e * (float)s + o * (float)c);
}

// ---- dispatch ------------------------------------------------------------------------------------------------
template <typename T, int OP>
int launch_unary(const void* xv, void* yv, int64_t n, hipStream_t s) {
  const T* x = static_cast<const T*>(xv);
  T* y = static_cast<T*>(yv);
  constexpr int N = 16 / sizeof(T);
  if (aligned_to(x, 16) && aligned_to(y, 16) && n >= N) {
    const int64_t chunks = n / N;
    const int64_t blocks = (chunks + kEwThreads * kEwChunks - 1) / (kEwThreads * kEwChunks);
    if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((unary_kernel<T, OP>), dim3((unsigned)blocks), dim3(kEwThreads), 0, s, x, y, n);
  } else {
    const int64_t blocks = (n + kEwThreads - 1) / kEwThreads;
    if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((unary_scalar_kernel<T, OP>), dim3((unsigned)blocks), dim3(kEwThreads), 0, s, x, y, n);
  }
  return launch_status();
}

template <typename T>
int dispatch_unary(int op, const void* x, void* y, int64_t n, hipStream_t s) {
  switch (op) {
    case HEXMI_GELU_TANH: return launch_unary<T, HEXMI_GELU_TANH>(x, y, n, s);
    case HEXMI_SILU: return launch_unary<T, HEXMI_SILU>(x, y, n, s);
    case HEXMI_RSQRT: return launch_unary<T, HEXMI_RSQRT>(x, y, n, s);
    case HEXMI_SIN: return launch_unary<T, HEXMI_SIN>(x, y, n, s);
    case HEXMI_COS: return launch_unary<T, HEXMI_COS>(x, y, n, s);
    case HEXMI_EXP: return launch_unary<T, HEXMI_EXP>(x, y, n, s);
    default: return HEXMI_EINVAL;
  }
}

template <typename T, int OP>
int launch_binary(const void* av, const void* bv, void* yv, int64_t n, hipStream_t s) {
  const T* a = static_cast<const T*>(av);
  const T* b = static_cast<const T*>(bv);
  T* y = static_cast<T*>(yv);
  constexpr int N = 16 / sizeof(T);
  if (aligned_to(a, 16) && aligned_to(b, 16) && aligned_to(y, 16) && n >= N) {
    const int64_t chunks = n / N;
    const int64_t per_block = kEwThreads * kBinChunks;
    const int64_t blocks = (chunks + per_block - 1) / per_block;
    if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((binary_kernel<T, OP>), dim3((unsigned)blocks), dim3(kEwThreads), 0, s, a, b, y, n);
  } else {
    const int64_t blocks = (n + kEwThreads - 1) / kEwThreads;
    if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((binary_scalar_kernel<T, OP>), dim3((unsigned)blocks), dim3(kEwThreads), 0, s, a, b, y, n);
  }
  return launch_status();
}

template <typename T>
int dispatch_binary(int op, const void* a, const void* b, void* y, int64_t n, hipStream_t s) {
  switch (op) {
    case HEXMI_ADD: return launch_binary<T, HEXMI_ADD>(a, b, y, n, s);
    case HEXMI_SUB: return launch_binary<T, HEXMI_SUB>(a, b, y, n, s);
    case HEXMI_MUL: return launch_binary<T, HEXMI_MUL>(a, b, y, n, s);
    case HEXMI_DIV: return launch_binary<T, HEXMI_DIV>(a, b, y, n, s);
    default: return HEXMI_EINVAL;
  }
}

template <typename T, typename TOut>
int launch_block_sum_pass(const T* x, TOut* out, int64_t n, int64_t block, hipStream_t s) {
  const int64_t programs = (n + block - 1) / block;
  if (programs > 0x7fffffff) return HEXMI_ENOTSUP;
  if (block * (int64_t)sizeof(T) <= 65536)
    hipLaunchKernelGGL((block_sum_kernel<T, TOut, 256>), dim3((unsigned)programs), dim3(256), 0, s, x, out, block, n);
  else
    hipLaunchKernelGGL((block_sum_kernel<T, TOut, 1024>), dim3((unsigned)programs), dim3(1024), 0, s, x, out, block, n);
  return launch_status();
}

// partials == nullptr: one pass. Otherwise partials holds at least ceil(n / kSumRun) floats and two_pass_sum(n, block).
template <typename T>
int launch_block_sum(const void* xv, void* outv, int64_t n, int64_t block, float* partials, hipStream_t s) {
  const T* x = static_cast<const T*>(xv);
  T* out = static_cast<T*>(outv);
  if (!partials) return launch_block_sum_pass<T, T>(x, out, n, block, s);
  const int64_t runs = (n + kSumRun - 1) / kSumRun;
  const int rc = launch_block_sum_pass<T, float>(x, partials, n, kSumRun, s);
  if (rc != HEXMI_OK) return rc;
  return launch_block_sum_pass<float, T>(partials, out, runs, block >= n ? runs : block / kSumRun, s);
}

template <typename T>
int launch_rope(const void* xv, void* yv, int64_t batch, int64_t seq, int64_t heads, int64_t feat, double theta,
                hipStream_t s) {
  const T* x = static_cast<const T*>(xv);
  T* y = static_cast<T*>(yv);
  constexpr int N = 16 / sizeof(T);
  const double log2_theta = log2(theta);
  if (aligned_to(x, 16) && aligned_to(y, 16) && feat % N == 0 && feat / N <= 256 && batch * heads < 0x40000000) {
    // enough workgroups to fill the chip when the sequence is short: split the (batch, head) rows over grid.y
    const int64_t passes = (batch * heads + 256 / (feat / N) - 1) / (256 / (feat / N));
    int64_t split = (2048 + seq - 1) / seq;
    split = split < passes ? split : passes;
    split = split < 65535 ? split : 65535;
    hipLaunchKernelGGL((rope_kernel<T>), dim3((unsigned)seq, (unsigned)split), dim3(256), 0, s, x, y, (int)batch,
                       (int)seq, (int)heads, (int)feat, log2_theta, exp2(-2.0 * log2_theta / (double)feat));
  } else {
    const int64_t pairs = batch * seq * heads * (feat / 2);
    const int64_t blocks = (pairs + 255) / 256;
    if (blocks > 0x7fffffff) return HEXMI_ENOTSUP;
    hipLaunchKernelGGL((rope_pair_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, s, x, y, pairs, (int)seq,
                       (int)heads, (int)feat, log2_theta);
  }
  return launch_status();
}

// Out-of-place transpose of a matrix of 16-bit elements (bit patterns: fp16 and bf16 alike): 64 x 64 tiles through
// LDS, rows of the source read and rows of the destination written as contiguous runs, the LDS pitch odd in 32-bit
// words so neither side conflicts. Any shape and leading dimensions.
__global__ __launch_bounds__(256)
void transpose16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int rows, int cols,
                        int64_t ld_src, int64_t ld_dst) {
  __shared__ uint16_t tile[64][66];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = r0 + ty + 4 * i, c = c0 + tx;
    tile[ty + 4 * i][tx] = (r < rows && c < cols) ? src[(int64_t)r * ld_src + c] : (uint16_t)0;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int c = c0 + ty + 4 * i, r = r0 + tx;         // destination row c, column r
    if (c < cols && r < rows) dst[(int64_t)c * ld_dst + r] = tile[tx][ty + 4 * i];
  }
}

}  // namespace

int block_sum_any(const void* x, void* out, int64_t n, int64_t block, int dtype, float* partials, hipStream_t s) {
  switch (dtype) {
    case HEXMI_F32: return launch_block_sum<float>(x, out, n, block, partials, s);
    case HEXMI_F16: return launch_block_sum<f16>(x, out, n, block, partials, s);
    case HEXMI_BF16: return launch_block_sum<bf16>(x, out, n, block, partials, s);
    default: return HEXMI_ENOTSUP;
  }
}

}  // namespace hexmi

using namespace hexmi;

extern "C" int hexmi_unary(int op, const void* x, void* y, int64_t n, int dtype, hexmi_stream_t stream) {
  if (n < 0 || op < 0 || op > HEXMI_EXP) return HEXMI_EINVAL;
  if (n == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  hipStream_t s = as_stream(stream);
  begin_call();
  switch (dtype) {
    case HEXMI_F32: return dispatch_unary<float>(op, x, y, n, s);
    case HEXMI_F16: return dispatch_unary<f16>(op, x, y, n, s);
    case HEXMI_BF16: return dispatch_unary<bf16>(op, x, y, n, s);
    default: return HEXMI_ENOTSUP;
  }
}

extern "C" int hexmi_binary(int op, const void* a, const void* b, void* y, int64_t n, int dtype,
                            hexmi_stream_t stream) {
  if (n < 0 || op < 0 || op > HEXMI_DIV) return HEXMI_EINVAL;
  if (n == 0) return HEXMI_OK;
  if (!a || !b || !y) return HEXMI_EINVAL;
  hipStream_t s = as_stream(stream);
  begin_call();
  switch (dtype) {
    case HEXMI_F32: return dispatch_binary<float>(op, a, b, y, n, s);
    case HEXMI_F16: return dispatch_binary<f16>(op, a, b, y, n, s);
    case HEXMI_BF16: return dispatch_binary<bf16>(op, a, b, y, n, s);
    default: return HEXMI_ENOTSUP;
  }
}

extern "C" int hexmi_block_sum(const void* x, void* out, int64_t n, int64_t block, int dtype,
                               hexmi_stream_t stream) {
  return hexmi_block_sum_ws(x, out, n, block, dtype, nullptr, 0, stream);
}

extern "C" int64_t hexmi_block_sum_workspace(int64_t n, int64_t block, int dtype) {
  (void)dtype;
  if (n <= 0 || block <= 0 || !two_pass_sum(n, block)) return 0;
  return (n + kSumRun - 1) / kSumRun * (int64_t)sizeof(float);
}

extern "C" int hexmi_block_sum_ws(const void* x, void* out, int64_t n, int64_t block, int dtype, void* workspace,
                                  int64_t workspace_bytes, hexmi_stream_t stream) {
  if (n < 0 || block <= 0 || workspace_bytes < 0) return HEXMI_EINVAL;
  if (n == 0) return HEXMI_OK;
  if (!x || !out) return HEXMI_EINVAL;
  float* partials = nullptr;
  if (workspace && two_pass_sum(n, block)) {
    if (workspace_bytes < hexmi_block_sum_workspace(n, block, dtype) || !aligned_to(workspace, 4)) return HEXMI_EINVAL;
    partials = static_cast<float*>(workspace);
  }
  begin_call();
  return block_sum_any(x, out, n, block, dtype, partials, as_stream(stream));
}

extern "C" int hexmi_rope(const void* x, void* y, int64_t batch, int64_t seq, int64_t heads, int64_t feat,
                          double theta, int dtype, hexmi_stream_t stream) {
  if (batch < 0 || seq < 0 || heads < 0 || feat < 0 || feat % 2 != 0 || !(theta > 0.0)) return HEXMI_EINVAL;
  if (batch == 0 || seq == 0 || heads == 0 || feat == 0) return HEXMI_OK;
  if (!x || !y) return HEXMI_EINVAL;
  if (batch > 0x7fffffff || seq > 0x7fffffff || heads > 0x7fffffff || feat > 0x7fffffff) return HEXMI_ENOTSUP;
  hipStream_t s = as_stream(stream);
  begin_call();
  switch (dtype) {
    case HEXMI_F32: return launch_rope<float>(x, y, batch, seq, heads, feat, theta, s);
    case HEXMI_F16: return launch_rope<f16>(x, y, batch, seq, heads, feat, theta, s);
    case HEXMI_BF16: return launch_rope<bf16>(x, y, batch, seq, heads, feat, theta, s);
    default: return HEXMI_ENOTSUP;
  }
}

extern "C" int hexmi_transpose16(int64_t rows, int64_t cols, const void* src, int64_t ld_src, void* dst, int64_t ld_dst,
                                 hexmi_stream_t stream) {
  if (rows < 0 || cols < 0) return HEXMI_EINVAL;
  if (rows == 0 || cols == 0) return HEXMI_OK;
  if (!src || !dst || ld_src < cols || ld_dst < rows) return HEXMI_EINVAL;
  const int64_t gx = (cols + 63) / 64, gy = (rows + 63) / 64;
  if (rows > 0x7fffffff || cols > 0x7fffffff || gy > 65535) return HEXMI_ENOTSUP;
  begin_call();
  hipLaunchKernelGGL(transpose16_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, as_stream(stream),
                     static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), (int)rows, (int)cols, ld_src, ld_dst);
  return launch_status();
}
