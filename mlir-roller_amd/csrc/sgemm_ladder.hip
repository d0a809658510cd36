// Teaching ladder: ten fp32 kernels for C = A*B + 1 on gfx950, from one thread per element to the
// matrix cores.  Counterpart of the tutorial kernels in /root/reference/src/cuda_matmul_opt.py:321-875
// (same kernel names, same "+1" payload, same static shapes), written for 64-lane wavefronts; the
// last two rungs (wave tiling on 64 lanes, MFMA) have no equivalent there.
//
// Shapes are compile-time, as in the reference (its kernels are generic over M, K, N and
// instantiated per size): -DM= -DK= -DN= are mandatory, and so is -DRUNG=<1..10>, which selects the
// one kernel a translation unit contains (the rungs share tile-parameter names with different
// meanings and constraints).  No kernel checks bounds; the host side
// refuses sizes that a rung's tiles do not divide.  Row-major operands; the *_transpose_B rung
// takes B as Bt[N][K].
//
// rung                                         what it teaches
//  1 sgemm_naive                               x walks rows: every lane of a wave touches another row
//  2 sgemm_naive_row_order                     x walks columns: B and C accesses of a wave coalesce
//  3 sgemm_coalesce                            the same from a linear thread id
//  4 sgemm_coalesce_transpose_B                both operands K-contiguous (no gain by itself)
//  5 sgemm_shared_mem_block                    BLOCK x BLOCK tiles through LDS: 1/BLOCK the global reads
//  6 sgemm_shared_mem_1d_block_tiling          TM results per thread: one LDS read of B feeds TM FMAs
//  7 sgemm_shared_mem_2d_block_tiling          TM x TN results per thread: outer product from registers
//  8 sgemm_shared_mem_2d_block_tiling_vectorize  128-bit global and LDS accesses, A transposed in LDS
//  9 sgemm_wave_tiling                         a wave owns a WM x WN sub-tile: LDS reads broadcast inside it
// 10 sgemm_mfma                                v_mfma_f32_32x32x2_f32 straight from global memory

#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

#if !defined(M) || !defined(K) || !defined(N) || !defined(RUNG)
#error "define the problem size and the rung to build: -DM=.. -DK=.. -DN=.. -DRUNG=1..10"
#endif

#ifndef BLOCK      /* rungs 1-5: edge of the square thread block / tile */
#define BLOCK 32
#endif
#ifndef BM         /* rungs 6-9: block tile */
#define BM 64
#endif
#ifndef BN
#define BN 64
#endif
#ifndef BK
#define BK 8
#endif
#ifndef TM         /* rungs 6-9: results per thread */
#define TM 8
#endif
#ifndef TN
#define TN 8
#endif
#ifndef WM         /* rung 9: wave tile and its column passes */
#define WM 64
#endif
#ifndef WN
#define WN 64
#endif
#ifndef WNITER
#define WNITER 2
#endif

#define WAVE 64
#define GLOBAL extern "C" __global__

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16 __attribute__((ext_vector_type(16)));

static __device__ __forceinline__ int linear_tid() { return threadIdx.y * blockDim.x + threadIdx.x; }

// ---- 1, 2: one thread per element, (BLOCK, BLOCK) threads per block -------------------------------

#if RUNG == 1
GLOBAL void sgemm_naive(const float* A, const float* B, float* C) {
  const int r = blockDim.x * blockIdx.x + threadIdx.x;   // neighbouring lanes: neighbouring ROWS
  const int c = blockDim.y * blockIdx.y + threadIdx.y;
  float sum = 0.0f;
  for (int k = 0; k < K; ++k) sum += A[r * K + k] * B[k * N + c];
  C[r * N + c] = sum + 1.0f;
}
#endif

#if RUNG == 2
GLOBAL void sgemm_naive_row_order(const float* A, const float* B, float* C) {
  const int c = blockDim.x * blockIdx.x + threadIdx.x;   // neighbouring lanes: neighbouring COLUMNS
  const int r = blockDim.y * blockIdx.y + threadIdx.y;
  float sum = 0.0f;
  for (int k = 0; k < K; ++k) sum += A[r * K + k] * B[k * N + c];
  C[r * N + c] = sum + 1.0f;
}
#endif

// ---- 3, 4: BLOCK*BLOCK threads, position derived from the linear id -------------------------------

#if RUNG == 3
GLOBAL void sgemm_coalesce(const float* A, const float* B, float* C) {
  const int t = linear_tid();
  const int r = blockIdx.x * BLOCK + t / BLOCK;
  const int c = blockIdx.y * BLOCK + t % BLOCK;
  float sum = 0.0f;
  for (int k = 0; k < K; ++k) sum += A[r * K + k] * B[k * N + c];
  C[r * N + c] = sum + 1.0f;
}
#endif

#if RUNG == 4
GLOBAL void sgemm_coalesce_transpose_B(const float* A, const float* Bt, float* C) {
  const int t = linear_tid();
  const int r = blockIdx.x * BLOCK + t / BLOCK;
  const int c = blockIdx.y * BLOCK + t % BLOCK;
  float sum = 0.0f;
  for (int k = 0; k < K; ++k) sum += A[r * K + k] * Bt[c * K + k];
  C[r * N + c] = sum + 1.0f;
}
#endif

// ---- 5: square tiles through LDS -------------------------------------------------------------------

#if RUNG == 5
GLOBAL void sgemm_shared_mem_block(const float* A, const float* B, float* C) {
  extern __shared__ float lds[];
  float* As = lds;                   // [BLOCK][BLOCK]
  float* Bs = lds + BLOCK * BLOCK;   // [BLOCK][BLOCK]
  const int t = linear_tid();
  const int tr = t / BLOCK, tc = t % BLOCK;
  const int row0 = blockIdx.x * BLOCK, col0 = blockIdx.y * BLOCK;
  float sum = 0.0f;
  for (int k0 = 0; k0 < K; k0 += BLOCK) {
    As[tr * BLOCK + tc] = A[(row0 + tr) * K + k0 + tc];
    Bs[tr * BLOCK + tc] = B[(k0 + tr) * N + col0 + tc];
    __syncthreads();
    for (int k = 0; k < BLOCK; ++k) sum += As[tr * BLOCK + k] * Bs[k * BLOCK + tc];
    __syncthreads();
  }
  C[(row0 + tr) * N + col0 + tc] = sum + 1.0f;
}
#endif

// ---- 6: a column of TM results per thread; (BM/TM)*BN threads --------------------------------------

#if RUNG == 6
GLOBAL void sgemm_shared_mem_1d_block_tiling(const float* A, const float* B, float* C) {
  constexpr int NT = (BM / TM) * BN;
  static_assert(BM * BK == NT && BK * BN == NT, "one element of each operand tile per thread");
  extern __shared__ float lds[];
  float* As = lds;             // [BM][BK]
  float* Bs = lds + BM * BK;   // [BK][BN]
  const int t = linear_tid();
  const int tc = t % BN, tr = t / BN;
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
  float acc[TM] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
    As[t] = A[(row0 + t / BK) * K + k0 + t % BK];
    Bs[t] = B[(k0 + t / BN) * N + col0 + t % BN];
    __syncthreads();
    for (int k = 0; k < BK; ++k) {
      const float b = Bs[k * BN + tc];
#pragma unroll
      for (int i = 0; i < TM; ++i) acc[i] += As[(tr * TM + i) * BK + k] * b;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) C[(row0 + tr * TM + i) * N + col0 + tc] = acc[i] + 1.0f;
}
#endif

// ---- 7: TM x TN results per thread; (BM/TM)*(BN/TN) threads ----------------------------------------

#if RUNG == 7
GLOBAL void sgemm_shared_mem_2d_block_tiling(const float* A, const float* B, float* C) {
  constexpr int NT = (BM / TM) * (BN / TN);
  extern __shared__ float lds[];
  float* As = lds;             // [BM][BK]
  float* Bs = lds + BM * BK;   // [BK][BN]
  const int t = linear_tid();
  const int tc = t % (BN / TN), tr = t / (BN / TN);
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
  float acc[TM][TN] = {};
  float a[TM], b[TN];
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int e = t; e < BM * BK; e += NT) As[e] = A[(row0 + e / BK) * K + k0 + e % BK];
    for (int e = t; e < BK * BN; e += NT) Bs[e] = B[(k0 + e / BN) * N + col0 + e % BN];
    __syncthreads();
    for (int k = 0; k < BK; ++k) {
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[(tr * TM + i) * BK + k];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Bs[k * BN + tc * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) C[(row0 + tr * TM + i) * N + col0 + tc * TN + j] = acc[i][j] + 1.0f;
}
#endif

// ---- 8: the same with 128-bit accesses; A is transposed on its way into LDS ------------------------

#if RUNG == 8
GLOBAL void sgemm_shared_mem_2d_block_tiling_vectorize(const float* A, const float* B, float* C) {
  constexpr int NT = (BM / TM) * (BN / TN);
  static_assert(BK % 4 == 0 && BN % 4 == 0 && TN % 4 == 0 && K % 4 == 0 && N % 4 == 0, "128-bit accesses");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* As = lds;             // [BK][BM]: reading TM consecutive rows of one k is then contiguous
  float* Bs = lds + BM * BK;   // [BK][BN]
  const int t = linear_tid();
  const int tc = t % (BN / TN), tr = t / (BN / TN);
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
  float acc[TM][TN] = {};
  float a[TM], b[TN];
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int u = t; u < BM * BK / 4; u += NT) {
      const int r = u / (BK / 4), c4 = (u % (BK / 4)) * 4;
      const f4 v = *(const f4*)&A[(row0 + r) * K + k0 + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) As[(c4 + j) * BM + r] = v[j];
    }
    for (int u = t; u < BK * BN / 4; u += NT) {
      const int r = u / (BN / 4), c4 = (u % (BN / 4)) * 4;
      *(f4*)&Bs[r * BN + c4] = *(const f4*)&B[(k0 + r) * N + col0 + c4];
    }
    __syncthreads();
    for (int k = 0; k < BK; ++k) {
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[k * BM + tr * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = Bs[k * BN + tc * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; j += 4) {
      const f4 out = {acc[i][j] + 1.0f, acc[i][j + 1] + 1.0f, acc[i][j + 2] + 1.0f, acc[i][j + 3] + 1.0f};
      *(f4*)&C[(row0 + tr * TM + i) * N + col0 + tc * TN + j] = out;
    }
}
#endif

// ---- 9: wave tiling for 64 lanes; (BM/WM)*(BN/WN) waves --------------------------------------------
// A wave owns WM x WN; it covers that area in WMITER x WNITER passes of a WSUBM x WSUBN sub-tile in
// which every lane holds TM x TN results.  All 64 lanes of a wave read LDS addresses that differ
// only inside the sub-tile, so most reads are broadcasts.

#if RUNG == 9
GLOBAL void sgemm_wave_tiling(const float* A, const float* B, float* C) {
  constexpr int NT = (BM / WM) * (BN / WN) * WAVE;
  constexpr int WMITER = (WM * WN) / (WAVE * TM * TN * WNITER);
  constexpr int WSUBM = WM / WMITER, WSUBN = WN / WNITER;
  static_assert(WMITER >= 1 && WMITER * WAVE * TM * TN * WNITER == WM * WN, "passes must tile the wave tile");
  static_assert((WSUBM / TM) * (WSUBN / TN) == WAVE, "64 lanes span one sub-tile");
  static_assert(BK % 4 == 0 && BN % 4 == 0 && TN % 4 == 0 && K % 4 == 0 && N % 4 == 0, "128-bit accesses");
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* As = lds;             // [BK][BM]
  float* Bs = lds + BM * BK;   // [BK][BN]
  const int t = linear_tid();
  const int wave = t / WAVE, lane = t % WAVE;
  const int wrow = (wave / (BN / WN)) * WM, wcol = (wave % (BN / WN)) * WN;
  const int lc = lane % (WSUBN / TN), lr = lane / (WSUBN / TN);
  const int row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;
  float acc[WMITER * TM][WNITER * TN] = {};
  float a[WMITER][TM], b[WNITER][TN];
  for (int k0 = 0; k0 < K; k0 += BK) {
    for (int u = t; u < BM * BK / 4; u += NT) {
      const int r = u / (BK / 4), c4 = (u % (BK / 4)) * 4;
      const f4 v = *(const f4*)&A[(row0 + r) * K + k0 + c4];
#pragma unroll
      for (int j = 0; j < 4; ++j) As[(c4 + j) * BM + r] = v[j];
    }
    for (int u = t; u < BK * BN / 4; u += NT) {
      const int r = u / (BN / 4), c4 = (u % (BN / 4)) * 4;
      *(f4*)&Bs[r * BN + c4] = *(const f4*)&B[(k0 + r) * N + col0 + c4];
    }
    __syncthreads();
    for (int k = 0; k < BK; ++k) {
#pragma unroll
      for (int wi = 0; wi < WMITER; ++wi)
#pragma unroll
        for (int i = 0; i < TM; ++i) a[wi][i] = As[k * BM + wrow + wi * WSUBM + lr * TM + i];
#pragma unroll
      for (int wj = 0; wj < WNITER; ++wj)
#pragma unroll
        for (int j = 0; j < TN; ++j) b[wj][j] = Bs[k * BN + wcol + wj * WSUBN + lc * TN + j];
#pragma unroll
      for (int wi = 0; wi < WMITER; ++wi)
#pragma unroll
        for (int wj = 0; wj < WNITER; ++wj)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[wi * TM + i][wj * TN + j] += a[wi][i] * b[wj][j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int wi = 0; wi < WMITER; ++wi)
#pragma unroll
    for (int wj = 0; wj < WNITER; ++wj)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; j += 4) {
          const int r = row0 + wrow + wi * WSUBM + lr * TM + i;
          const int c = col0 + wcol + wj * WSUBN + lc * TN + j;
          const float* s = &acc[wi * TM + i][wj * TN + j];
          const f4 out = {s[0] + 1.0f, s[1] + 1.0f, s[2] + 1.0f, s[3] + 1.0f};
          *(f4*)&C[r * N + c] = out;
        }
}
#endif

// ---- 10: the matrix cores, as plainly as possible ---------------------------------------------------
// 256 threads = 2 x 2 waves, one 32x32 block of C per wave, operands straight from global memory.
// v_mfma_f32_32x32x2_f32: lane l supplies A[row l%32][k + l/32] and B[k + l/32][col l%32]; result
// register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the block.

#if RUNG == 10
GLOBAL void sgemm_mfma(const float* A, const float* B, float* C) {
  static_assert(K % 2 == 0, "the instruction contracts two k at a time");
  const int t = linear_tid();
  const int wave = t / WAVE, lane = t % WAVE;
  const int row0 = blockIdx.y * 64 + (wave / 2) * 32, col0 = blockIdx.x * 64 + (wave % 2) * 32;
  const int i = lane % 32, g = lane / 32;
  f16 acc = {};
  for (int k = 0; k < K; k += 2)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(A[(row0 + i) * K + k + g], B[(k + g) * N + col0 + i], acc, 0, 0, 0);
#pragma unroll
  for (int r = 0; r < 16; ++r) C[(row0 + 8 * (r / 4) + 4 * g + r % 4) * N + col0 + i] = acc[r] + 1.0f;
}
#endif
