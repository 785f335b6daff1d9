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
#include "chol_leaf.hpp"

namespace ak {

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

// One work group (16 waves) per matrix: the n x n (n <= LEAF) diagonal block at `lo`, padded with an identity to
// a power-of-two multiple of 16, is factored in LDS by the recursion above: 16 x 16 blocks in the registers of one
// wave, everything else as 16x16x4 fp32 MFMA products over all waves.  On exit the block holds L^-1 in its lower
// triangle and zeros above the diagonal.
static __global__ __launch_bounds__(LEAF_THREADS) void chol_leaf_kernel(float* __restrict__ W, int64_t strideW,
                                                                        int64_t d, int lo, int n,
                                                                        int* __restrict__ info, const int* active,
                                                                        int active_stride) {
  extern __shared__ __attribute__((aligned(16))) float leaf_smem[];
  const int z = blockIdx.x;
  if (active != nullptr && active[static_cast<int64_t>(z) * active_stride] == 0) return;
  const int tid = threadIdx.x;
  leaf_block(W + z * strideW + static_cast<int64_t>(lo) * d + lo, d, n, leaf_smem, tid);
  const int bad = leaf_bad_pivot(leaf_smem);
  if (tid == 0 && bad != 0 && bad <= n && info[z] == 0) info[z] = lo + bad;
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
