// LDS-resident Cholesky factorization + triangular inverse of one diagonal block of at most 128 x 128, shared by
// the batched (one size) and the grouped (many sizes) damped inverse: 16 x 16 blocks are factored and inverted in
// the registers of one wave (v_readlane broadcasts), everything larger is the same recursion as the global one
//   T1 = A21 M11^T,  A22 -= T1 T1^T,  factor(A22),  M21 = -M22 (T1 M11)
// on LDS operands with v_mfma_f32_16x16x4_f32 tiles spread over the 16 waves of the work group.
#pragma once
#include "common.hpp"

namespace ak {

constexpr int LEAF = 128;

__device__ __forceinline__ float lane_bcast(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), src_lane));
}

constexpr int PB = 16;              // base block handled in registers by one wave
constexpr int LLD = LEAF + 4;       // LDS leading dimension: rows 4 banks apart, so the [row][k] operand reads of the
                                    // 16x16x4 MFMA (16 rows x 4 k per instruction) touch 64 different banks
constexpr int LEAF_THREADS = 1024;
constexpr int LEAF_WAVES = LEAF_THREADS / 64;
constexpr int T1_LD = 68;
// work block, T1 pool (64x64 + 32x32 + 16x16 panels of nested levels) and T2, plus the bad-pivot word
constexpr int LEAF_T1_FLOATS = 64 * T1_LD + 32 * T1_LD + 16 * T1_LD;
constexpr int LEAF_T2_FLOATS = 64 * T1_LD;
constexpr size_t LEAF_LDS_BYTES = (LEAF * LLD + LEAF_T1_FLOATS + LEAF_T2_FLOATS + 8) * sizeof(float);

// Cholesky factor and its inverse of a PB x PB block held one row per lane (lanes >= PB carry an identity
// row).  On exit a[] is row `lane` of L (entries right of the diagonal are meaningless) and m[] is row `lane` of
// L^-1 (zeros right of the diagonal).  Returns 0 or the 1-based index of the first non-positive pivot.
//
// One loop over the pivots does both.  Row i of the inverse is (e_i - sum_{k<i} l_ik m_k) / l_ii; every lane keeps the
// numerator u_i of its own row, and pivot k, whose row u_k is complete by then, subtracts (l_ik / l_kk) u_k from the
// rows below it: k + 1 lane reads and as many multiply-adds that do not depend on one another, next to the 15 - k of
// the factorization's own update, so that every pivot issues the same 16 + 16 and the wait states of the serial
// pivot chain (lane read, reciprocal square root, scaling, lane read, multiply-add) are filled.  A forward
// substitution after the factorization costs the same arithmetic as chains of up to 15 dependent multiply-adds,
// and took as long again as the factorization.
// Every step is applied to all lanes without masks where that is harmless: entries above the diagonal and the rows
// that are already final only ever receive values nobody reads (each broadcast below takes a[k] of a lane j >= k);
// the rows of the inverse are protected by a factor that is zero for the lanes at and above the pivot.
__device__ __forceinline__ int small_chol_inv(float (&a)[PB], float (&m)[PB], int lane) {
  int bad = 0;
  float my_inv = 1.f;
#pragma unroll
  for (int j = 0; j < PB; ++j) m[j] = (j == lane) ? 1.f : 0.f;
#pragma unroll
  for (int k = 0; k < PB; ++k) {
    float akk = lane_bcast(a[k], k);
    if (!(akk > 0.f)) {             // also catches NaN
      if (bad == 0) bad = k + 1;
      akk = 1.f;
    }
    float inv = __builtin_amdgcn_rsqf(akk);                 // hardware rsqrt, then one Newton step:
    inv = inv * (1.5f - 0.5f * akk * inv * inv);             // keeps the serial pivot chain short
    my_inv = (lane == k) ? inv : my_inv;
    a[k] *= inv;                    // lane k: a_kk / sqrt(a_kk) = l_kk; lanes below: l_ik
    const float f = (lane > k) ? a[k] * inv : 0.f;          // l_ik / l_kk for the rows below the pivot
    float l[PB], u[PB];
#pragma unroll
    for (int j = k + 1; j < PB; ++j) l[j] = lane_bcast(a[k], j);
#pragma unroll
    for (int j = 0; j <= k; ++j) u[j] = lane_bcast(m[j], k);
#pragma unroll
    for (int j = k + 1; j < PB; ++j) a[j] -= a[k] * l[j];
#pragma unroll
    for (int j = 0; j <= k; ++j) m[j] -= f * u[j];
  }
#pragma unroll
  for (int j = 0; j < PB; ++j) m[j] *= my_inv;
  return bad;
}

// v_mfma_f32_16x16x4_f32: lane l feeds A[i = l%16][k = l/16] and B[k = l/16][j = l%16]; accumulator register r of
// lane l is C[i = 4*(l/16) + r][j = l%16].
__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Which part of the contraction range a 16x16 output tile (ib, jb) needs when one operand is triangular (the rest
// multiplies zeros).
enum LeafK { LK_FULL, LK_LE_J, LK_GE_J, LK_LE_I };

// C[M x N] (=, -=) alpha * A[M x K] * op(B) for small matrices in LDS, all sizes multiples of 16, one 16x16 output
// tile per wave and turn.  TB: op(B)[k][j] = B[j][k].  LOWER: only tiles on or below the diagonal (M == N).
// ACC: C -= product, else C = alpha * product.  The caller synchronises before and after.
template <int M, int N, int K, bool TB, bool LOWER, bool ACC, LeafK KM>
__device__ __forceinline__ void leaf_gemm(float* __restrict__ C, int ldc, const float* __restrict__ A, int lda,
                                          const float* __restrict__ B, int ldb, float alpha, int wave, int lane) {
  constexpr int TM = M / 16, TN = N / 16;
  const int li = lane & 15, lk = lane >> 4;
#pragma unroll 1
  for (int t = wave; t < TM * TN; t += LEAF_WAVES) {
    const int ib = t / TN, jb = t % TN;
    if (LOWER && jb > ib) continue;
    // The whole contraction range, whatever KM says: the triangular operands hold zeros outside their triangle, and
    // a loop whose bounds depend on the tile waits for the LDS once per step (the recursion is a chain of some thirty
    // of these products, each as long as its slowest tile).  Here every operand of the tile is requested before
    // the first matrix instruction is issued.
    constexpr int KS = K / 4;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    const float* pa = A + (16 * ib + li) * lda + lk;
    const float* pb = TB ? B + (16 * jb + li) * ldb + lk : B + lk * ldb + 16 * jb + li;
    float av[KS], bv[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      av[s] = pa[4 * s];
      bv[s] = TB ? pb[4 * s] : pb[4 * s * ldb];
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) acc = mfma16(av[s], bv[s], acc);
    float* pc = C + (16 * ib + 4 * lk) * ldc + 16 * jb + li;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (ACC) pc[r * ldc] -= acc[r];
      else pc[r * ldc] = alpha * acc[r];
    }
  }
}

// Factors the N x N block of Wm at (lo, lo) and leaves the inverse of its Cholesky factor in the lower triangle;
// same recursion as the global one, on LDS operands.  t1: this level's slice of the T1 pool.
template <int N>
__device__ __forceinline__ void leaf_factor(float* __restrict__ Wm, int lo, float* __restrict__ t1,
                                            float* __restrict__ t2, int* __restrict__ s_bad, int tid) {
  const int wave = tid >> 6, lane = tid & 63;
  if constexpr (N == PB) {
    if (wave == 0) {
      float a[PB], m[PB];
      // every lane reads a whole row (the lanes beyond the block re-read its last one) with four 16-byte loads that
      // are all in flight together; a load under a per-element condition would be waited for on its own
      const floatx4* row = reinterpret_cast<const floatx4*>(Wm + (lo + (lane < PB ? lane : PB - 1)) * LLD + lo);
      floatx4 q[PB / 4];
#pragma unroll
      for (int c = 0; c < PB / 4; ++c) q[c] = row[c];
#pragma unroll
      for (int j = 0; j < PB; ++j) a[j] = (lane < PB && j <= lane) ? q[j >> 2][j & 3] : ((j == lane) ? 1.f : 0.f);
      const int bad = small_chol_inv(a, m, lane);
      if (lane < PB) {
        floatx4* dst = reinterpret_cast<floatx4*>(Wm + (lo + lane) * LLD + lo);
#pragma unroll
        for (int c = 0; c < PB / 4; ++c) {
          const floatx4 w = {m[4 * c], m[4 * c + 1], m[4 * c + 2], m[4 * c + 3]};     // zeros above the diagonal
          dst[c] = w;
        }
      }
      if (lane == 0 && bad != 0 && *s_bad == 0) *s_bad = lo + bad;
    }
    __syncthreads();
  } else {
    constexpr int H = N / 2;
    leaf_factor<H>(Wm, lo, t1, t2, s_bad, tid);
    float* W11 = Wm + lo * LLD + lo;
    float* W21 = Wm + (lo + H) * LLD + lo;
    float* W22 = Wm + (lo + H) * LLD + lo + H;
    leaf_gemm<H, H, H, true, false, false, LK_LE_J>(t1, T1_LD, W21, LLD, W11, LLD, 1.f, wave, lane);   // T1 = A21 M11^T
    __syncthreads();
    leaf_gemm<H, H, H, true, true, true, LK_FULL>(W22, LLD, t1, T1_LD, t1, T1_LD, 1.f, wave, lane);    // A22 -= T1 T1^T
    __syncthreads();
    leaf_factor<H>(Wm, lo + H, t1 + H * T1_LD, t2, s_bad, tid);
    leaf_gemm<H, H, H, false, false, false, LK_GE_J>(t2, T1_LD, t1, T1_LD, W11, LLD, 1.f, wave, lane); // T2 = T1 M11
    __syncthreads();
    leaf_gemm<H, H, H, false, false, false, LK_LE_I>(W21, LLD, W22, LLD, t2, T1_LD, -1.f, wave, lane); // M21 = -M22 T2
    __syncthreads();
  }
}


// Loads the n x n block at `blk` (row stride ld), padded with an identity to npad in {16, 32, 64, 128}, factors it
// in the LDS and writes L^-1 back (lower triangle, zeros above the diagonal).  Returns in *s_bad the 1-based index
// of the first non-positive pivot inside the block, or 0.  All 1024 threads of the work group call it.
__device__ __forceinline__ void leaf_block(float* __restrict__ blk, int64_t ld, int n, float* leaf_smem, int tid) {
  float* Wm = leaf_smem;
  float* t1 = leaf_smem + LEAF * LLD;
  float* t2 = t1 + LEAF_T1_FLOATS;
  int* s_bad = reinterpret_cast<int*>(t2 + LEAF_T2_FLOATS);
  const int npad = n <= 16 ? 16 : (n <= 32 ? 32 : (n <= 64 ? 64 : 128));
  {
    // all of this thread's elements are requested before the first one is stored: a load and its store per turn
    // would pay the latency of the device memory sixteen times over
    constexpr int ROWS_PER_TURN = LEAF_THREADS / 128, TURNS = LEAF / ROWS_PER_TURN;
    const int j = tid & 127;
    float v[TURNS];
#pragma unroll
    for (int t = 0; t < TURNS; ++t) {
      const int i = (tid >> 7) + ROWS_PER_TURN * t;
      v[t] = (i == j) ? 1.f : 0.f;                 // identity padding beyond n
      if (i < n && j < n) v[t] = (j <= i) ? blk[static_cast<int64_t>(i) * ld + j] : 0.f;
    }
#pragma unroll
    for (int t = 0; t < TURNS; ++t) {
      const int i = (tid >> 7) + ROWS_PER_TURN * t;
      if (i < npad && j < npad) Wm[i * LLD + j] = v[t];
    }
  }
  if (tid == 0) *s_bad = 0;
  __syncthreads();
  if (npad == 16) leaf_factor<16>(Wm, 0, t1, t2, s_bad, tid);
  else if (npad == 32) leaf_factor<32>(Wm, 0, t1, t2, s_bad, tid);
  else if (npad == 64) leaf_factor<64>(Wm, 0, t1, t2, s_bad, tid);
  else leaf_factor<128>(Wm, 0, t1, t2, s_bad, tid);
  for (int i = tid >> 7; i < n; i += LEAF_THREADS / 128) {
    const int j = tid & 127;
    if (j < n) blk[static_cast<int64_t>(i) * ld + j] = (j <= i) ? Wm[i * LLD + j] : 0.f;
  }
}

__device__ __forceinline__ int leaf_bad_pivot(const float* leaf_smem) {
  return *reinterpret_cast<const int*>(leaf_smem + LEAF * LLD + LEAF_T1_FLOATS + LEAF_T2_FLOATS);
}

}  // namespace ak
