// Dense fp32 products exposed through the C ABI: the general GEMM and the Kronecker
// preconditioning G <- grad_scale * Binv G Ainv (+ bias <- grad_scale * Binv bias).
#include <mutex>
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

// The same for many matrices in one launch.  `table`: one row of 5 int64 per product: M, x, y, n, first block
// (blocks of 4 rows, numbered in table order); y must not alias x.
static __global__ __launch_bounds__(256) void gemv_grouped_kernel(const int64_t* __restrict__ table, int count,
                                                                  float scale) {
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * 5 + 4] <= w) lo = mid;
    else hi = mid - 1;
  }
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * 5;
  const float* __restrict__ M = reinterpret_cast<const float*>(r[0]);
  const float* __restrict__ x = reinterpret_cast<const float*>(r[1]);
  float* __restrict__ y = reinterpret_cast<float*>(r[2]);
  const int64_t n = r[3];
  const int64_t row = static_cast<int64_t>(w - r[4]) * 4 + (threadIdx.x >> 6);
  if (row >= n) return;
  const int lane = threadIdx.x & 63;
  float s = 0.f;
  for (int64_t k = lane; k < n; k += 64) s += M[row * n + k] * x[k];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) y[row] = scale * s;
}

// Convolution weight gradients between the channels-last layout [Cout][kh*kw][Cin] and the contiguous layout
// [Cout][Cin][kh*kw] the Kronecker factors are indexed by, for many modules in one launch: one work group per
// output channel stages the row in the LDS, so both the read and the write are coalesced.  `table`: one row of
// 5 int64 per module: channels-last address, contiguous address, Cin, kh*kw, first row (running sum of Cout).
constexpr int LAYOUT_MAX_ROW = 12288;       // floats of one weight row (Cin * kh * kw) the staging buffer holds

static __global__ __launch_bounds__(256) void weight_layout_grouped_kernel(const int64_t* __restrict__ table, int count,
                                                                           int to_contiguous) {
  __shared__ float row[LAYOUT_MAX_ROW];
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * 5 + 4] <= w) lo = mid;
    else hi = mid - 1;
  }
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * 5;
  const int cin = static_cast<int>(r[2]), kk = static_cast<int>(r[3]);
  const int len = cin * kk;
  const int64_t off = static_cast<int64_t>(w - r[4]) * len;
  float* nhwc = reinterpret_cast<float*>(r[0]) + off;
  float* nchw = reinterpret_cast<float*>(r[1]) + off;
  const float* __restrict__ src = to_contiguous ? nhwc : nchw;
  float* __restrict__ dst = to_contiguous ? nchw : nhwc;
  for (int i = threadIdx.x; i < len; i += 256) row[i] = src[i];
  __syncthreads();
  if (to_contiguous) {
    for (int n = threadIdx.x; n < len; n += 256) dst[n] = row[(n % kk) * cin + n / kk];      // n = ci * kk + k
  } else {
    for (int j = threadIdx.x; j < len; j += 256) dst[j] = row[(j % cin) * kk + j / cin];     // j = k * cin + ci
  }
}

// Largest magnitudes of many strided vectors in one launch.  `table`: one row of 5 int64 per vector: address, number
// of elements, element stride, address of the float word the maximum is folded into (integer atomic maximum on the
// bit pattern; the caller zeroes the words first), first block (blocks of ABSMAX_BLOCK elements, numbered in table order).
constexpr int ABSMAX_BLOCK = 8192;

static __global__ __launch_bounds__(256) void absmax_grouped_kernel(const int64_t* __restrict__ table, int count) {
  __shared__ float red[4];
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * 5 + 4] <= w) lo = mid;
    else hi = mid - 1;
  }
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * 5;
  const float* __restrict__ x = reinterpret_cast<const float*>(r[0]);
  const int64_t n = r[1], stride = r[2];
  const int64_t i0 = static_cast<int64_t>(w - r[4]) * ABSMAX_BLOCK;
  const int64_t i1 = i0 + ABSMAX_BLOCK < n ? i0 + ABSMAX_BLOCK : n;
  float m = 0.f;
  if (stride == 1 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
    const int64_t iv = i0 + ((i1 - i0) & ~static_cast<int64_t>(3));      // i0 is a multiple of 4
    for (int64_t i = i0 + 4 * threadIdx.x; i < iv; i += 1024) {
      const floatx4 v = *reinterpret_cast<const floatx4*>(x + i);
      m = fmaxf(fmaxf(m, fmaxf(fabsf(v[0]), fabsf(v[1]))), fmaxf(fabsf(v[2]), fabsf(v[3])));
    }
    for (int64_t i = iv + threadIdx.x; i < i1; i += 256) m = fmaxf(m, fabsf(x[i]));      // the ragged end of the vector
  } else {
    for (int64_t i = i0 + threadIdx.x; i < i1; i += 256) m = fmaxf(m, fabsf(x[i * stride]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    atomicMax(reinterpret_cast<unsigned int*>(r[3]), __builtin_bit_cast(unsigned int, m));
  }
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

namespace ak {

// G <- grad_scale * Binv G Ainv through the intermediate T = [dB, dA] (+ dB floats behind it for the bias).
static int kron_precond_run(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA, float* bias,
                            float grad_scale, float* T, hipStream_t s) {
  const int b = static_cast<int>(dB), a = static_cast<int>(dA);
  // the inverses are symmetric: reading A^-1 as its transpose makes both operands of the second product
  // contiguous along the contraction index
  GemmParams g1 = make_gemm(0, 0, b, a, b, 1.f, Binv, dB, G, dA, 0.f, T, dA);
  GemmParams g2 = make_gemm(0, 1, b, a, a, grad_scale, T, dA, Ainv, dA, 0.f, G, dA);
  g1.split = g2.split = 3;
  int rc = launch_gemm(g1, 1, s);
  if (rc != AK_OK) return rc;
  rc = launch_gemm(g2, 1, s);
  if (rc != AK_OK) return rc;
  if (bias != nullptr) {
    float* tb = T + dB * dA;
    hipLaunchKernelGGL(gemv_kernel, dim3(static_cast<unsigned>((dB + 3) / 4)), dim3(256), 0, s, Binv, bias, tb, dB,
                       grad_scale);
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<unsigned>((dB + 255) / 256)), dim3(256), 0, s, tb, bias, dB);
  }
  return check_launch();
}

// Intermediate of ak_kron_precond_static: one array per GPU, held from the first call on that GPU until the process
// ends.  In host code `scratch` is only a handle for hipGetSymbolAddress; kernels get the address looked up below.
constexpr int64_t STATIC_SCRATCH_FLOATS = 4ll << 20;      // 16 MiB
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static float* g_scratch_ptr[MAX_DEVICES];                 // device address of `scratch` on each GPU, null until looked up

// Address of the current device's copy of `scratch` (looked up once per device, with that device current).
static int static_scratch(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return AK_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    float* ptr = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr)
      return AK_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return AK_OK;
}

}  // namespace ak

extern "C" int ak_kron_precond(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA, float* bias,
                               float grad_scale, void* ws, size_t ws_bytes, ak_stream_t stream) {
  if (Binv == nullptr || Ainv == nullptr || G == nullptr || dB <= 0 || dA <= 0 || dB > (1 << 30) || dA > (1 << 30))
    return AK_ERR_ARG;
  if (ws == nullptr || ws_bytes < ak_kron_precond_ws_bytes(dB, dA)) return AK_ERR_WORKSPACE;
  return ak::kron_precond_run(Binv, Ainv, G, dB, dA, bias, grad_scale, static_cast<float*>(ws),
                              static_cast<hipStream_t>(stream));
}

extern "C" int64_t ak_kron_precond_static_max_floats(void) { return ak::STATIC_SCRATCH_FLOATS; }

extern "C" int ak_kron_precond_static(const float* Binv, const float* Ainv, float* G, int64_t dB, int64_t dA,
                                      float* bias, float grad_scale, ak_stream_t stream) {
  if (Binv == nullptr || Ainv == nullptr || G == nullptr || dB <= 0 || dA <= 0 || dB > (1 << 30) || dA > (1 << 30))
    return AK_ERR_ARG;
  if (dB * dA + dB > ak::STATIC_SCRATCH_FLOATS) return AK_ERR_TOO_LARGE;
  float* T = nullptr;
  const int rc = ak::static_scratch(&T);
  if (rc != AK_OK) return rc;
  // both products overwrite their whole output without reading it, so what the last call left in T does not matter
  return ak::kron_precond_run(Binv, Ainv, G, dB, dA, bias, grad_scale, T, static_cast<hipStream_t>(stream));
}

extern "C" int ak_gemm_f32_grouped(int pieces, const int64_t* table, int count, int64_t total_tiles,
                                   ak_stream_t stream) {
  if (pieces != 0 && pieces != 2 && pieces != 3 && pieces != 22 && pieces != 23) return AK_ERR_ARG;
  if (count < 0 || total_tiles < 0 || total_tiles > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_tiles == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(total_tiles));
  if (pieces == 0) hipLaunchKernelGGL(ak::gemm_f32_grouped_kernel, grid, dim3(256), 0, s, table, count);
  else if (pieces == 2) hipLaunchKernelGGL(ak::gemm_x3_grouped_kernel<2>, grid, dim3(256), 0, s, table, count);
  else if (pieces == 22) hipLaunchKernelGGL((ak::gemm_x3_grouped_kernel<2, true>), grid, dim3(256), 0, s, table, count);
  else if (pieces == 23) hipLaunchKernelGGL((ak::gemm_x3_grouped_kernel<2, true, true>), grid, dim3(256), 0, s, table, count);
  else hipLaunchKernelGGL(ak::gemm_x3_grouped_kernel<3>, grid, dim3(256), 0, s, table, count);
  return ak::check_launch();
}

extern "C" int ak_gemv_f32_grouped(const int64_t* table, int count, int64_t total_blocks, float alpha,
                                   ak_stream_t stream) {
  if (count < 0 || total_blocks < 0 || total_blocks > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_blocks == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::gemv_grouped_kernel, dim3(static_cast<unsigned>(total_blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), table, count, alpha);
  return ak::check_launch();
}

extern "C" int64_t ak_absmax_block(void) { return ak::ABSMAX_BLOCK; }

extern "C" int ak_absmax_grouped(const int64_t* table, int count, int64_t total_blocks, ak_stream_t stream) {
  if (count < 0 || total_blocks < 0 || total_blocks > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_blocks == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::absmax_grouped_kernel, dim3(static_cast<unsigned>(total_blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), table, count);
  return ak::check_launch();
}

extern "C" int64_t ak_weight_layout_max_row(void) { return ak::LAYOUT_MAX_ROW; }

extern "C" int ak_weight_layout_grouped(const int64_t* table, int count, int64_t total_rows, int to_contiguous,
                                        ak_stream_t stream) {
  if (count < 0 || total_rows < 0 || total_rows > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_rows == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::weight_layout_grouped_kernel, dim3(static_cast<unsigned>(total_rows)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), table, count, to_contiguous != 0 ? 1 : 0);
  return ak::check_launch();
}

#ifdef AK_TUNING_HOOKS
// Tuning builds only (-DAK_TUNING_HOOKS): the smallest grid (in 128 x 128 tiles) and contraction length from which
// products that ask for the split-bf16 kernel get it.
extern "C" void ak_debug_set_gemm_split_threshold(int min_groups, int min_k) {
  ak::g_x3_min_groups = min_groups;
  ak::g_x3_min_k = min_k;
}

extern "C" void ak_debug_set_gemm_double_buffer(int on) { ak::g_x3_double_buffer = on; }
#endif
