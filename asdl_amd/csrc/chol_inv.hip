// out <- (A + lam I)^-1 for a batch of same-size symmetric positive definite fp32 matrices.
//
// Recursive blocked Cholesky that carries the triangular inverse along:
//   F(lo, hi): n <= 128 -> one work group factors the block in LDS and inverts the factor.
//              otherwise, with [lo,mid) / [mid,hi) and M11 = L11^-1 already in place,
//                T1  = A21 M11^T            (= L21; the triangular solve is a product)
//                A22 -= T1 T1^T             (lower triangle only)
//                F(mid, hi)
//                M21 = -M22 (T1 M11)
// so that the lower triangle of the work matrix ends up holding M = L^-1, and
//   out = M^T M  (contraction restricted to k >= max(i, j), mirrored to both triangles).
// All panel and trailing updates are fp32 MFMA GEMM tiles whose contraction range skips the
// zero half of the triangular operand.  The order of launches is fixed by d alone, so the
// whole inverse is enqueued without any host synchronisation; a non positive definite
// pivot is reported through the device `info` word (LAPACK potrf convention).
#include "gemm_f32.hpp"

namespace ak {

constexpr int LEAF = 128;

struct BatchPtrs {
  const float* const* A_list;
  const int* active;
  int active_stride;
};

// W_z <- lower(A_z) + lam_z I, strict upper triangle zero.  grid (ceil(d/16), ceil(d/64), batch), 256 threads.
static __global__ __launch_bounds__(256) void chol_copy_in_kernel(BatchPtrs bp, float* __restrict__ W, int64_t strideW,
                                                                  int64_t d, const float* __restrict__ lam,
                                                                  int lam_stride, int* __restrict__ info) {
  const int z = blockIdx.z;
  if (bp.active != nullptr && bp.active[static_cast<int64_t>(z) * bp.active_stride] == 0) return;
  const float* __restrict__ A = bp.A_list[z];
  const int64_t col = static_cast<int64_t>(blockIdx.y) * 64 + (threadIdx.x & 63);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 16 + (threadIdx.x >> 6) * 4;
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) info[z] = 0;
  if (col >= d) return;
  const float l = lam[static_cast<int64_t>(z) * lam_stride];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int64_t r = row + e;
    if (r >= d) break;
    float v = 0.f;
    if (col <= r) v = A[r * d + col];
    if (col == r) v += l;
    W[z * strideW + r * d + col] = v;
  }
}

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
// row).  On exit a[] is row `lane` of L and m[] is column `lane` of L^-1.  Returns 0 or the 1-based index of
// the first non-positive pivot.
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
    const float lkk = akk * inv;
    inv_diag[k] = inv;
    a[k] = (lane > k) ? a[k] * inv : ((lane == k) ? lkk : a[k]);
#pragma unroll
    for (int j = k + 1; j < PB; ++j) {
      const float ljk = lane_bcast(a[k], j);
      a[j] = (lane >= j) ? a[j] - a[k] * ljk : a[j];
    }
  }
#pragma unroll
  for (int i = 0; i < PB; ++i) {   // column `lane` of L^-1 by forward substitution down the rows
    float s = (lane == i) ? 1.f : 0.f;
#pragma unroll
    for (int k = 0; k < i; ++k) s -= lane_bcast(a[k], i) * m[k];
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

// One work group (16 waves) per matrix: the n x n (n <= LEAF) diagonal block at `lo`, padded with an identity to
// a power-of-two multiple of 16, is factored in LDS by the recursion above: 16 x 16 blocks in the registers of one
// wave, everything else as 16x16x4 fp32 MFMA products over all waves.  On exit the block holds L^-1 in its lower
// triangle and zeros above the diagonal.
static __global__ __launch_bounds__(LEAF_THREADS) void chol_leaf_kernel(float* __restrict__ W, int64_t strideW,
                                                                        int64_t d, int lo, int n,
                                                                        int* __restrict__ info, const int* active,
                                                                        int active_stride) {
  extern __shared__ __attribute__((aligned(16))) float leaf_smem[];
  float* Wm = leaf_smem;
  float* t1 = leaf_smem + LEAF * LLD;
  float* t2 = t1 + LEAF_T1_FLOATS;
  int* s_bad = reinterpret_cast<int*>(t2 + LEAF_T2_FLOATS);
  const int z = blockIdx.x;
  if (active != nullptr && active[static_cast<int64_t>(z) * active_stride] == 0) return;
  const int tid = threadIdx.x;
  const int npad = n <= 16 ? 16 : (n <= 32 ? 32 : (n <= 64 ? 64 : 128));
  float* __restrict__ blk = W + z * strideW + static_cast<int64_t>(lo) * d + lo;
  for (int i = tid >> 7; i < npad; i += LEAF_THREADS / 128) {
    const int j = tid & 127;
    if (j < npad) {
      float v = (i == j) ? 1.f : 0.f;              // identity padding beyond n
      if (i < n && j < n) v = (j <= i) ? blk[static_cast<int64_t>(i) * d + j] : 0.f;
      Wm[i * LLD + j] = v;
    }
  }
  if (tid == 0) *s_bad = 0;
  __syncthreads();
  if (npad == 16) leaf_factor<16>(Wm, 0, t1, t2, s_bad, tid);
  else if (npad == 32) leaf_factor<32>(Wm, 0, t1, t2, s_bad, tid);
  else if (npad == 64) leaf_factor<64>(Wm, 0, t1, t2, s_bad, tid);
  else leaf_factor<128>(Wm, 0, t1, t2, s_bad, tid);
  if (tid == 0 && *s_bad != 0 && *s_bad <= n && info[z] == 0) info[z] = lo + *s_bad;
  for (int i = tid >> 7; i < n; i += LEAF_THREADS / 128) {
    const int j = tid & 127;
    if (j < n) blk[static_cast<int64_t>(i) * d + j] = (j <= i) ? Wm[i * LLD + j] : 0.f;
  }
}

struct CholCtx {
  float* W;
  float* T1;
  float* T2;
  int64_t d, strideW, strideT1, strideT2;
  int batch;
  int* info;
  const int* active;
  int active_stride;
  hipStream_t stream;
  int rc;
};

static void run_gemm(CholCtx& c, GemmParams p) {
  p.active = c.active;
  p.active_stride = c.active_stride;
  p.split = 3;          // large products run on the bf16 matrix cores with fp32-grade accuracy
  const int rc = launch_gemm(p, c.batch, c.stream);
  if (rc != AK_OK) c.rc = rc;
}

static void factor_range(CholCtx& c, int lo, int hi, int64_t t1_off) {
  const int n = hi - lo;
  if (n <= LEAF) {
    hipLaunchKernelGGL(chol_leaf_kernel, dim3(c.batch), dim3(LEAF_THREADS), LEAF_LDS_BYTES, c.stream, c.W, c.strideW,
                       c.d, lo, n, c.info, c.active, c.active_stride);
    return;
  }
  const int nb = (n + LEAF - 1) / LEAF;
  const int mid = lo + LEAF * ((nb + 1) / 2);
  factor_range(c, lo, mid, t1_off);
  float* T1 = c.T1 + t1_off;   // must survive the recursion into [mid, hi): that one allocates past it
  const int s1 = mid - lo, s2 = hi - mid;
  const int64_t d = c.d;
  float* W11 = c.W + static_cast<int64_t>(lo) * d + lo;
  float* W21 = c.W + static_cast<int64_t>(mid) * d + lo;
  float* W22 = c.W + static_cast<int64_t>(mid) * d + mid;
  {  // T1 = A21 M11^T
    GemmParams p = make_gemm(0, 1, s2, s1, s1, 1.f, W21, d, W11, d, 0.f, T1, s1);
    p.sA = c.strideW; p.sB = c.strideW; p.sC = c.strideT1; p.kmode = K_LE_J;
    run_gemm(c, p);
  }
  {  // A22 -= T1 T1^T
    GemmParams p = make_gemm(0, 1, s2, s2, s1, -1.f, T1, s1, T1, s1, 1.f, W22, d);
    p.sA = c.strideT1; p.sB = c.strideT1; p.sC = c.strideW; p.tile_mode = TILE_LOWER;
    run_gemm(c, p);
  }
  factor_range(c, mid, hi, t1_off + static_cast<int64_t>(s1) * s2);
  {  // T2 = T1 M11
    GemmParams p = make_gemm(0, 0, s2, s1, s1, 1.f, T1, s1, W11, d, 0.f, c.T2, s1);
    p.sA = c.strideT1; p.sB = c.strideW; p.sC = c.strideT2; p.kmode = K_GE_J;
    run_gemm(c, p);
  }
  {  // M21 = -M22 T2
    GemmParams p = make_gemm(0, 0, s2, s1, s2, -1.f, W22, d, c.T2, s1, 0.f, W21, d);
    p.sA = c.strideW; p.sB = c.strideT2; p.sC = c.strideW; p.kmode = K_LE_I;
    run_gemm(c, p);
  }
}

static int64_t half_size(int64_t d) {
  const int64_t nb = (d + LEAF - 1) / LEAF;
  return LEAF * ((nb + 1) / 2);
}

// Elements of the T1 pool one matrix needs: a node's panel lives while its right half is factored.
static int64_t t1_pool_size(int64_t n) {
  if (n <= LEAF) return 0;
  const int64_t s1 = half_size(n), s2 = n - s1;
  const int64_t left = t1_pool_size(s1), right = s1 * s2 + t1_pool_size(s2);
  return left > right ? left : right;
}

}  // namespace ak

extern "C" size_t ak_chol_inv_ws_bytes(int64_t d, int batch) {
  if (d <= 0 || batch <= 0) return 0;
  const int64_t h = ak::half_size(d);
  return static_cast<size_t>(batch) * (d * d + h * h + ak::t1_pool_size(d)) * sizeof(float);
}

extern "C" int ak_chol_inv_batched(const float* const* A_list, float* const* out_list, int64_t d, int batch,
                                   const float* lam, int lam_stride, const int* skip_flags, int skip_stride, int* info,
                                   void* ws, size_t ws_bytes, ak_stream_t stream) {
  using namespace ak;
  if (A_list == nullptr || out_list == nullptr || lam == nullptr || info == nullptr || d <= 0 || batch <= 0 ||
      d > (1 << 20))
    return AK_ERR_ARG;
  if (ws == nullptr || ws_bytes < ak_chol_inv_ws_bytes(d, batch)) return AK_ERR_WORKSPACE;
  const int64_t h = half_size(d);
  CholCtx c;
  c.W = static_cast<float*>(ws);
  c.T1 = c.W + static_cast<int64_t>(batch) * d * d;
  const int64_t pool = t1_pool_size(d);
  c.T2 = c.T1 + static_cast<int64_t>(batch) * pool;
  c.d = d; c.strideW = d * d; c.strideT1 = pool; c.strideT2 = h * h;
  c.batch = batch; c.info = info;
  c.active = skip_flags; c.active_stride = skip_stride;
  c.stream = static_cast<hipStream_t>(stream);
  c.rc = AK_OK;
  static bool leaf_attr_set = false;     // idempotent; a benign race sets it twice at worst
  if (!leaf_attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(chol_leaf_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(LEAF_LDS_BYTES)) != hipSuccess)
      return AK_ERR_LAUNCH;
    leaf_attr_set = true;
  }
  BatchPtrs bp{A_list, skip_flags, skip_stride};
  dim3 grid(static_cast<unsigned>((d + 15) / 16), static_cast<unsigned>((d + 63) / 64), batch);
  hipLaunchKernelGGL(chol_copy_in_kernel, grid, dim3(256), 0, c.stream, bp, c.W, c.strideW, d, lam, lam_stride, info);
  factor_range(c, 0, static_cast<int>(d), 0);
  {  // out = M^T M
    GemmParams p = make_gemm(1, 0, static_cast<int>(d), static_cast<int>(d), static_cast<int>(d), 1.f, c.W, d, c.W, d,
                             0.f, nullptr, d);
    p.C_list = out_list;
    p.sA = c.strideW; p.sB = c.strideW; p.kmode = K_GE_MAXIJ; p.tile_mode = TILE_LOWER_MIRROR;
    run_gemm(c, p);
  }
  if (c.rc != AK_OK) return c.rc;
  return check_launch();
}
