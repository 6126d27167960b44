// fp32 GEMM on the matrix cores: C[M,N] = A[M,K] B[K,N] (or A B^T with B [N,K]) with fp32 operands and
// v_mfma_f32_32x32x2_f32, no rounding of the operands (the fp32 matmuls of the reference's torch-mlir graphs,
// test/python/torch-mlir/test_add_matmul_softmax.py:25-29, at any size). 157 TFLOP/s is the part's fp32 matrix
// peak; the vector-ALU kernel in gemm.hip stays for the shapes this one does not take (K % 32 != 0, unaligned
// operands).
//
// A workgroup of four waves owns a 128 x 128 tile (64 x 64 per wave: four 32 x 32 accumulators), K walks in slabs of
// 32 (128-byte rows: whole L2 lines), two LDS stages per operand, two workgroups per CU. A slab is 64 MFMAs of 64
// cycles per wave, far longer than the memory latency, so plain double buffering (copy slab s+1 while slab s is
// multiplied, one barrier per slab) keeps the matrix cores fed. Copies are buffer loads into LDS (copy_to_lds).
// Products with fewer than one such tile per CU take 64 x 64 tiles (one accumulator per wave): four times the
// workgroups, each through its K loop four times as fast.
//
// LDS layouts (16-byte chunks, swizzled through the copies' source addresses):
//   K-contiguous operand (A, and B when it is [N,K]): [128 rows][8 chunks], chunk ^ (row/2)%8. A lane reads one
//     chunk (4 consecutive k) of its row with ds_read_b128 and feeds 4 MFMAs from it: the MFMA's two k slots are
//     assigned to k = 8q + e (lanes 0..31) and 8q + 4 + e (lanes 32..63), e = 0..3.
//   N-contiguous operand (B as [K,N]): [32 k][32 chunks], chunk ^ 8*((k/4)%2). A lane reads B[k][n] with
//     ds_read_b32; the two k slots of an MFMA are 4 apart, so the swizzle puts the two half-waves on disjoint banks.
#include "hexmi_common.h"

namespace hexmi {
namespace {

constexpr int kSlabK = 32;       // K per slab

typedef float f32x4v __attribute__((ext_vector_type(4)));

// WT: 32 x 32 accumulators per wave along each side (2: 128 x 128 workgroup tile, 1: 64 x 64)
template <bool TRANS_B, int WT>
__global__ __launch_bounds__(256, WT == 2 ? 2 : 4)
void gemm_f32_mfma_kernel(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C, int M,
                          int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int tiles_m, int tiles_n) {
  constexpr int kTile = 64 * WT;                     // rows and columns of the workgroup tile
  constexpr int NI = kTile * 8 / 64 / 4;             // copy instructions per wave, operand and slab
  __shared__ __attribute__((aligned(16))) float a_s0[kTile * kSlabK];
  __shared__ __attribute__((aligned(16))) float a_s1[kTile * kSlabK];
  __shared__ __attribute__((aligned(16))) float b_s0[kTile * kSlabK];
  __shared__ __attribute__((aligned(16))) float b_s1[kTile * kSlabK];

  const int lane = threadIdx.x % kWave, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int wm = wave / 2, wn = wave % 2;
  // workgroup ids are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles (whole rows of the
  // tile grid when they divide evenly), so the A panels it streams stay in its L2
  const int tiles = tiles_m * tiles_n;
  int tile = blockIdx.x;
  if (tiles % 8 == 0) tile = (blockIdx.x % 8) * (tiles / 8) + blockIdx.x / 8;
  const int tm = tile / tiles_n, tn = tile % tiles_n;
  const int m0 = tm * kTile, n0 = tn * kTile;

  // ---- copies: kTile/8 wave-wide instructions per operand and slab, NI per wave
  const char* a_tile = reinterpret_cast<const char*>(A + (int64_t)m0 * lda);
  const char* b_tile = TRANS_B ? reinterpret_cast<const char*>(B + (int64_t)n0 * ldb)
                               : reinterpret_cast<const char*>(B + n0);
  int a_voff[NI], b_voff[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int q = j * 4 + wave;
    {
      const int row = q * 8 + lane / 8, pc = lane % 8;
      const int r = row < M - m0 ? row : M - m0 - 1;           // rows past the end repeat the last row
      a_voff[j] = (int)((r * lda + ((pc ^ ((row >> 1) & 7)) * 4)) * (int64_t)sizeof(float));
    }
    if (TRANS_B) {
      const int row = q * 8 + lane / 8, pc = lane % 8;
      const int r = row < N - n0 ? row : N - n0 - 1;
      b_voff[j] = (int)((r * ldb + ((pc ^ ((row >> 1) & 7)) * 4)) * (int64_t)sizeof(float));
    } else {
      constexpr int CPR = kTile / 4;                             // chunks per row of the [32 k][kTile n] tile
      const int k = q * (64 / CPR) + lane / CPR, pc = lane % CPR;
      int col = (pc ^ (((k >> 2) & 1) << 3)) * 4;
      col = n0 + col + 4 <= N ? col : N - 4 - n0;              // columns past the end repeat the last chunk
      b_voff[j] = (int)((k * ldb + col) * (int64_t)sizeof(float));
    }
  }
  auto issue = [&](int slab, float* a_dst, float* b_dst) __attribute__((always_inline)) {
    const char* a_src = a_tile + (int64_t)slab * kSlabK * sizeof(float);
    const char* b_src = TRANS_B ? b_tile + (int64_t)slab * kSlabK * sizeof(float)
                                : b_tile + (int64_t)slab * kSlabK * ldb * sizeof(float);
#pragma unroll
    for (int j = 0; j < NI; ++j) copy_to_lds(a_src, a_voff[j], a_dst + (j * 4 + wave) * 256);
#pragma unroll
    for (int j = 0; j < NI; ++j) copy_to_lds(b_src, b_voff[j], b_dst + (j * 4 + wave) * 256);
  };

  // ---- fragments
  const int r32 = lane % 32, kh = lane / 32;
  int a_row[WT], b_row[WT];
#pragma unroll
  for (int i = 0; i < WT; ++i) {
    a_row[i] = wm * 32 * WT + i * 32 + r32;
    b_row[i] = wn * 32 * WT + i * 32 + r32;
  }
  f32x16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  auto multiply = [&](const float* as, const float* bs) __attribute__((always_inline)) {
#pragma unroll
    for (int kq = 0; kq < kSlabK / 8; ++kq) {
      f32x4v af[WT], bf[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i)
        af[i] = *reinterpret_cast<const f32x4v*>(as + a_row[i] * kSlabK + (((kq * 2 + kh) ^ ((a_row[i] >> 1) & 7)) * 4));
      if (TRANS_B) {
#pragma unroll
        for (int j = 0; j < WT; ++j)
          bf[j] = *reinterpret_cast<const f32x4v*>(bs + b_row[j] * kSlabK + (((kq * 2 + kh) ^ ((b_row[j] >> 1) & 7)) * 4));
      } else {
#pragma unroll
        for (int j = 0; j < WT; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            bf[j][e] = bs[(kq * 8 + kh * 4 + e) * kTile + (((b_row[j] >> 2) ^ (kh << 3)) * 4) + (b_row[j] & 3)];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < WT; ++i)
#pragma unroll
          for (int j = 0; j < WT; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
    }
  };

  const int n_slabs = K / kSlabK;
  issue(0, a_s0, b_s0);
  int s = 0;
  for (; s + 1 < n_slabs; s += 2) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    issue(s + 1, a_s1, b_s1);
    multiply(a_s0, b_s0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (s + 2 < n_slabs) issue(s + 2, a_s0, b_s0);
    multiply(a_s1, b_s1);
  }
  if (s < n_slabs) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    multiply(a_s0, b_s0);
  }

  // ---- acc[i][j][r] is C[m0 + (wm*WT + i)*32 + 8*(r/4) + 4*kh + r%4][n0 + (wn*WT + j)*32 + r32]
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j) {
      const int col = n0 + wn * 32 * WT + j * 32 + r32;
      if (col >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 32 * WT + i * 32 + 8 * (r / 4) + 4 * kh + r % 4;
        if (row < M) C[(int64_t)row * ldc + col] = acc[i][j][r];
      }
    }
}

}  // namespace

// True (and the product launched, status in *status) when the shapes fit this kernel: whole 32-wide slabs, 16-byte
// chunks that start on 16-byte boundaries, per-lane copy offsets below 2^31 bytes.
bool gemm_f32_mfma(bool trans_b, const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K,
                   int64_t lda, int64_t ldb, int64_t ldc, hipStream_t s, int* status) {
  if (K % kSlabK != 0 || lda % 4 != 0 || ldb % 4 != 0 || !aligned_to(A, 16) || !aligned_to(B, 16)) return false;
  if (!trans_b && (N % 4 != 0 || N < 4)) return false;
  if (lda >= (1 << 21) || ldb >= (1 << 21)) return false;
  const int cus = hexmi_num_cus();
  const int64_t big = ((M + 127) / 128) * ((N + 127) / 128);
  const int tile = big >= (cus > 0 ? cus : 256) ? 128 : 64;    // fewer than one 128 x 128 tile per CU: 64 x 64 tiles
  const int64_t tiles_m = (M + tile - 1) / tile, tiles_n = (N + tile - 1) / tile;
  if (tiles_m * tiles_n > 0x7fffffff) return false;
#define HEXMI_F32_MFMA(TB, WT) \
  hipLaunchKernelGGL((gemm_f32_mfma_kernel<TB, WT>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256), 0, s, A, B, C, \
                     (int)M, (int)N, (int)K, lda, ldb, ldc, (int)tiles_m, (int)tiles_n)
  if (trans_b) {
    if (tile == 128) HEXMI_F32_MFMA(true, 2); else HEXMI_F32_MFMA(true, 1);
  } else {
    if (tile == 128) HEXMI_F32_MFMA(false, 2); else HEXMI_F32_MFMA(false, 1);
  }
#undef HEXMI_F32_MFMA
  *status = launch_status();
  return true;
}

}  // namespace hexmi
