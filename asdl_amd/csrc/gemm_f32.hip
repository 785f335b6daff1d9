// Dense fp32 products exposed through the C ABI: the general GEMM and the Kronecker
// preconditioning G <- grad_scale * Binv G Ainv (+ bias <- grad_scale * Binv bias).
#include "gemm_f32.hpp"

namespace ak {

// y <- scale * M x for a dense row-major [n, n] matrix; one wave per row.  grid ceil(n/4), 256 threads.
static __global__ __launch_bounds__(256) void gemv_kernel(const float* __restrict__ M, const float* __restrict__ x,
                                                          float* __restrict__ y, int64_t n, float scale) {
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= n) return;
  const int lane = threadIdx.x & 63;
  float s = 0.f;
  for (int64_t k = lane; k < n; k += 64) s += M[row * n + k] * x[k];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) y[row] = scale * s;
}

static __global__ void copy_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

}  // namespace ak

extern "C" int ak_gemm_f32(int transA, int transB, int64_t M, int64_t N, int64_t K, float alpha, const float* A,
                           int64_t lda, const float* B, int64_t ldb, float beta, float* C, int64_t ldc, int batch,
                           int64_t strideA, int64_t strideB, int64_t strideC, ak_stream_t stream) {
  if (A == nullptr || B == nullptr || C == nullptr || M < 0 || N < 0 || K < 0 || batch <= 0) return AK_ERR_ARG;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return AK_ERR_ARG;
  const int64_t a_cols = transA ? M : K, b_cols = transB ? K : N;
  if (lda < a_cols || ldb < b_cols || ldc < N) return AK_ERR_ARG;
  ak::GemmParams p = ak::make_gemm(transA != 0, transB != 0, static_cast<int>(M), static_cast<int>(N),
                                   static_cast<int>(K), alpha, A, lda, B, ldb, beta, C, ldc);
  p.sA = strideA; p.sB = strideB; p.sC = strideC;
  return ak::launch_gemm(p, batch, static_cast<hipStream_t>(stream));
}

extern "C" int ak_gemm_f32_split(int pieces, int transA, int transB, int64_t M, int64_t N, int64_t K, float alpha,
                                 const float* A, int64_t lda, const float* B, int64_t ldb, float beta, float* C,
                                 int64_t ldc, int batch, int64_t strideA, int64_t strideB, int64_t strideC,
                                 ak_stream_t stream) {
  if (A == nullptr || B == nullptr || C == nullptr || M < 0 || N < 0 || K < 0 || batch <= 0) return AK_ERR_ARG;
  if (pieces != 0 && pieces != 2 && pieces != 3) return AK_ERR_ARG;
  if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30)) return AK_ERR_ARG;
  const int64_t a_cols = transA ? M : K, b_cols = transB ? K : N;
  if (lda < a_cols || ldb < b_cols || ldc < N) return AK_ERR_ARG;
  ak::GemmParams p = ak::make_gemm(transA != 0, transB != 0, static_cast<int>(M), static_cast<int>(N),
                                   static_cast<int>(K), alpha, A, lda, B, ldb, beta, C, ldc);
  p.sA = strideA; p.sB = strideB; p.sC = strideC;
  p.split = pieces;
  return ak::launch_gemm(p, batch, static_cast<hipStream_t>(stream));
}

extern "C" size_t ak_kron_precond_ws_bytes(int64_t dB, int64_t dA) {
  if (dB <= 0 || dA <= 0) return 0;
  return static_cast<size_t>(dB * dA + dB) * sizeof(float);
}

extern "C" int ak_kron_precond(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA, float* bias,
                               float grad_scale, void* ws, size_t ws_bytes, ak_stream_t stream) {
  if (Binv == nullptr || Ainv == nullptr || G == nullptr || dB <= 0 || dA <= 0 || dB > (1 << 30) || dA > (1 << 30))
    return AK_ERR_ARG;
  if (ws == nullptr || ws_bytes < ak_kron_precond_ws_bytes(dB, dA)) return AK_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* T = static_cast<float*>(ws);
  const int b = static_cast<int>(dB), a = static_cast<int>(dA);
  // the inverses are symmetric: reading A^-1 as its transpose makes both operands of the second product
  // contiguous along the contraction index
  ak::GemmParams g1 = ak::make_gemm(0, 0, b, a, b, 1.f, Binv, dB, G, dA, 0.f, T, dA);
  ak::GemmParams g2 = ak::make_gemm(0, 1, b, a, a, grad_scale, T, dA, Ainv, dA, 0.f, G, dA);
  g1.split = g2.split = 3;
  int rc = ak::launch_gemm(g1, 1, s);
  if (rc != AK_OK) return rc;
  rc = ak::launch_gemm(g2, 1, s);
  if (rc != AK_OK) return rc;
  if (bias != nullptr) {
    float* tb = T + dB * dA;
    hipLaunchKernelGGL(ak::gemv_kernel, dim3(static_cast<unsigned>((dB + 3) / 4)), dim3(256), 0, s, Binv, bias, tb, dB,
                       grad_scale);
    hipLaunchKernelGGL(ak::copy_kernel, dim3(static_cast<unsigned>((dB + 255) / 256)), dim3(256), 0, s, tb, bias, dB);
  }
  return ak::check_launch();
}

// Tuning hook, not part of the interface: the smallest grid (in 128 x 128 tiles) and contraction length from which
// products that ask for the split-bf16 kernel get it.
extern "C" void ak_debug_set_gemm_split_threshold(int min_groups, int min_k) {
  ak::g_x3_min_groups = min_groups;
  ak::g_x3_min_k = min_k;
}
