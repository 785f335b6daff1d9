// Kernels of the low-rank ("swift") Kronecker factors: when a layer sees fewer samples n than a factor has
// columns d, the factor is kept as the n x d matrix X of per-sample sums and (X^T X / n + lam I)^-1 is taken through
// the n x n Gram matrix (Sherman-Morrison-Woodbury).
//   patch_sum:  X[n][(c,ky,kx)] = sum over output positions of the patch element, straight from the activation
//               (kh = kw = 1: the sum over positions of an output gradient; H = W = 1: a scaled fp32 copy)
//   smw_finish: out = (I - Z) / lam with lam read from device memory
// All are bound by the HBM; the dense products in between run in the GEMM / SYRK / Cholesky kernels.
#include "common.hpp"

namespace ak {

struct PatchSumParams {
  const void* x;
  int64_t sn, sc, sh, sw;              // element strides of x[n][c][iy][ix]
  int N, C, H, W, kh, kw, strh, strw, ph, pw, Ho, Wo;
  float alpha, beta;
  float* out;                          // [N][C*kh*kw]
  int64_t ldo;
};

template <typename T>
__device__ __forceinline__ float ps_load(const T* p);
template <>
__device__ __forceinline__ float ps_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ps_load<uint16_t>(const uint16_t* p) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(*p) << 16);
}

// Channels innermost (NHWC memory): one thread per (tap, channel), lanes along the channels, so that every load of a
// wave is one contiguous run; the positions are walked serially.  grid (ceil(C / 64), kh*kw, N), 64 threads.
template <typename T>
static __global__ __launch_bounds__(64) void patch_sum_chan_kernel(PatchSumParams p) {
  const int c = blockIdx.x * 64 + threadIdx.x, tap = blockIdx.y, n = blockIdx.z;
  if (c >= p.C) return;
  const int ky = tap / p.kw, kx = tap - ky * p.kw;
  const T* __restrict__ base = static_cast<const T*>(p.x) + static_cast<int64_t>(n) * p.sn + static_cast<int64_t>(c) * p.sc;
  float s0 = 0.f, s1 = 0.f;
  for (int oy = 0; oy < p.Ho; ++oy) {
    const int iy = oy * p.strh + ky - p.ph;
    if (iy < 0 || iy >= p.H) continue;
    const T* __restrict__ row = base + static_cast<int64_t>(iy) * p.sh;
    int ox = 0;
    for (; ox + 1 < p.Wo; ox += 2) {
      const int ix0 = ox * p.strw + kx - p.pw, ix1 = ix0 + p.strw;
      if (ix0 >= 0 && ix0 < p.W) s0 += ps_load<T>(row + static_cast<int64_t>(ix0) * p.sw);
      if (ix1 >= 0 && ix1 < p.W) s1 += ps_load<T>(row + static_cast<int64_t>(ix1) * p.sw);
    }
    if (ox < p.Wo) {
      const int ix0 = ox * p.strw + kx - p.pw;
      if (ix0 >= 0 && ix0 < p.W) s0 += ps_load<T>(row + static_cast<int64_t>(ix0) * p.sw);
    }
  }
  float* dst = p.out + static_cast<int64_t>(n) * p.ldo + static_cast<int64_t>(c) * (p.kh * p.kw) + tap;
  float v = p.alpha * (s0 + s1);
  if (p.beta != 0.f) v += p.beta * *dst;
  *dst = v;
}

// Any other layout (NCHW: columns innermost): one wave per (n, c, tap), lanes along the output columns, rows walked
// serially, wave reduction at the end.  grid (kh*kw, C, N), 64 threads.
template <typename T>
static __global__ __launch_bounds__(64) void patch_sum_col_kernel(PatchSumParams p) {
  const int tap = blockIdx.x, c = blockIdx.y, n = blockIdx.z, lane = threadIdx.x;
  const int ky = tap / p.kw, kx = tap - ky * p.kw;
  const T* __restrict__ base = static_cast<const T*>(p.x) + static_cast<int64_t>(n) * p.sn + static_cast<int64_t>(c) * p.sc;
  float s = 0.f;
  for (int oy = 0; oy < p.Ho; ++oy) {
    const int iy = oy * p.strh + ky - p.ph;
    if (iy < 0 || iy >= p.H) continue;
    const T* __restrict__ row = base + static_cast<int64_t>(iy) * p.sh;
    for (int ox = lane; ox < p.Wo; ox += 64) {
      const int ix = ox * p.strw + kx - p.pw;
      if (ix >= 0 && ix < p.W) s += ps_load<T>(row + static_cast<int64_t>(ix) * p.sw);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if (lane == 0) {
    float* dst = p.out + static_cast<int64_t>(n) * p.ldo + static_cast<int64_t>(c) * (p.kh * p.kw) + tap;
    float v = p.alpha * s;
    if (p.beta != 0.f) v += p.beta * *dst;
    *dst = v;
  }
}

static __global__ __launch_bounds__(256) void smw_finish_kernel(float* __restrict__ Z, int64_t d, int64_t ld,
                                                                const float* __restrict__ lam) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, i = blockIdx.y;
  if (j >= d) return;
  const float inv = 1.f / lam[0];
  const float z = Z[i * ld + j];
  Z[i * ld + j] = ((i == j ? 1.f : 0.f) - z) * inv;
}

}  // namespace ak

extern "C" int ak_conv_patch_sum(const void* x, int dtype, int64_t sn, int64_t sc, int64_t sh_el, int64_t sw_el, int64_t N,
                                 int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw,
                                 float alpha, float beta, float* out, int64_t ldo, ak_stream_t stream) {
  if (x == nullptr || out == nullptr || N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 ||
      sw <= 0 || ph < 0 || pw < 0 || ldo < C * kh * kw)
    return AK_ERR_ARG;
  if (dtype != AK_BF16 && dtype != AK_F32) return AK_ERR_ARG;
  const int64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
  if (Ho <= 0 || Wo <= 0) return AK_ERR_ARG;
  if (N > 65535 || C > (1 << 24) || kh * kw > 65535 || H > (1 << 24) || W > (1 << 24)) return AK_ERR_UNSUPPORTED;
  ak::PatchSumParams p;
  p.x = x; p.sn = sn; p.sc = sc; p.sh = sh_el; p.sw = sw_el;
  p.N = static_cast<int>(N); p.C = static_cast<int>(C); p.H = static_cast<int>(H); p.W = static_cast<int>(W);
  p.kh = kh; p.kw = kw; p.strh = sh; p.strw = sw; p.ph = ph; p.pw = pw;
  p.Ho = static_cast<int>(Ho); p.Wo = static_cast<int>(Wo);
  p.alpha = alpha; p.beta = beta; p.out = out; p.ldo = ldo;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (sc == 1 && C > 1) {
    dim3 grid(static_cast<unsigned>((C + 63) / 64), kh * kw, static_cast<unsigned>(N));
    if (dtype == AK_BF16) hipLaunchKernelGGL(ak::patch_sum_chan_kernel<uint16_t>, grid, dim3(64), 0, s, p);
    else hipLaunchKernelGGL(ak::patch_sum_chan_kernel<float>, grid, dim3(64), 0, s, p);
  } else {
    if (C > 65535) return AK_ERR_UNSUPPORTED;
    dim3 grid(kh * kw, static_cast<unsigned>(C), static_cast<unsigned>(N));
    if (dtype == AK_BF16) hipLaunchKernelGGL(ak::patch_sum_col_kernel<uint16_t>, grid, dim3(64), 0, s, p);
    else hipLaunchKernelGGL(ak::patch_sum_col_kernel<float>, grid, dim3(64), 0, s, p);
  }
  return ak::check_launch();
}

extern "C" int ak_smw_finish(float* Z, int64_t d, int64_t ld, const float* lam, ak_stream_t stream) {
  if (Z == nullptr || lam == nullptr || d <= 0 || ld < d || d > 65535) return AK_ERR_ARG;
  dim3 grid(static_cast<unsigned>((d + 255) / 256), static_cast<unsigned>(d));
  hipLaunchKernelGGL(ak::smw_finish_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), Z, d, ld, lam);
  return ak::check_launch();
}
