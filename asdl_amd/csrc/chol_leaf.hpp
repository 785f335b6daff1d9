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
// row).  On exit a[] is row `lane` of L (entries right of the diagonal are meaningless) and m[] is column `lane`
// of L^-1.  Returns 0 or the 1-based index of the first non-positive pivot.
// Every step is applied to all lanes and all columns without masks: entries above the diagonal and the rows
// that are already final only ever receive values nobody reads (each broadcast below takes a[k] of a lane j >= k).
// The broadcasts of one pivot are issued together, ahead of the multiply-adds that use them, so that the wait
// states between a lane read and its first use are filled with the other lane reads.
__device__ __forceinline__ int small_chol_inv(float (&a)[PB], float (&m)[PB], int lane) {
  int bad = 0;
  float inv_diag[PB];
#pragma unroll
  for (int k = 0; k < PB; ++k) {
    float akk = lane_bcast(a[k], k);
    if (!(akk > 0.f)) {             // also catches NaN
      if (bad == 0) bad = k + 1;
      akk = 1.f;
    }
    float inv = __builtin_amdgcn_rsqf(akk);                 // hardware rsqrt, then one Newton step:
    inv = inv * (1.5f - 0.5f * akk * inv * inv);             // keeps the serial pivot chain short
    inv_diag[k] = inv;
    a[k] *= inv;                    // lane k: a_kk / sqrt(a_kk) = l_kk; lanes below: l_ik
    float l[PB];
#pragma unroll
    for (int j = k + 1; j < PB; ++j) l[j] = lane_bcast(a[k], j);
#pragma unroll
    for (int j = k + 1; j < PB; ++j) a[j] -= a[k] * l[j];
  }
#pragma unroll
  for (int i = 0; i < PB; ++i) {   // column `lane` of L^-1 by forward substitution down the rows
    float l[PB];
#pragma unroll
    for (int k = 0; k < i; ++k) l[k] = lane_bcast(a[k], i);
    float s = (lane == i) ? 1.f : 0.f;
#pragma unroll
    for (int k = 0; k < i; ++k) s -= l[k] * m[k];
    m[i] = (lane <= i) ? s * inv_diag[i] : 0.f;
  }
  return bad;
}

// v_mfma_f32_16x16x4_f32: lane l feeds A[i = l%16][k = l/16] and B[k = l/16][j = l%16]; accumulator register r of
// lane l is C[i = 4*(l/16) + r][j = l%16].
__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// Which part of the contraction range a 16x16 output tile (ib, jb) needs when one operand is triangular.
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
    int k0 = 0, k1 = K;
    if (KM == LK_LE_J) k1 = 16 * (jb + 1);
    if (KM == LK_GE_J) k0 = 16 * jb;
    if (KM == LK_LE_I) k1 = 16 * (ib + 1);
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    const float* pa = A + (16 * ib + li) * lda + lk;
    const float* pb = TB ? B + (16 * jb + li) * ldb + lk : B + lk * ldb + 16 * jb + li;
    for (int k = k0; k < k1; k += 4) {
      const float a = pa[k];
      const float b = TB ? pb[k] : pb[k * ldb];
      acc = mfma16(a, b, acc);
    }
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
#pragma unroll
      for (int j = 0; j < PB; ++j)
        a[j] = (lane < PB && j <= lane) ? Wm[(lo + lane) * LLD + lo + j] : ((j == lane) ? 1.f : 0.f);
      const int bad = small_chol_inv(a, m, lane);
      if (lane < PB) {
#pragma unroll
        for (int j = 0; j < PB; ++j) Wm[(lo + j) * LLD + lo + lane] = m[j];     // m[j] = 0 above the diagonal
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
  for (int i = tid >> 7; i < npad; i += LEAF_THREADS / 128) {
    const int j = tid & 127;
    if (j < npad) {
      float v = (i == j) ? 1.f : 0.f;              // identity padding beyond n
      if (i < n && j < n) v = (j <= i) ? blk[static_cast<int64_t>(i) * ld + j] : 0.f;
      Wm[i * LLD + j] = v;
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
