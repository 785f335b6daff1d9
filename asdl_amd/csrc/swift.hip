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

// Channels innermost (NHWC memory).  One work group per (tap, sample): thread t holds VEC consecutive channels
// (chunk t % CCH) and walks over the output positions t / CCH, t / CCH + PS, ... (PS = 256 / CCH position slices),
// so that a wave reads whole runs of channels with 16-byte loads (VEC = 8, bf16) and many positions are in flight;
// the slices are summed through LDS at the end.  grid (kh*kw, N, ceil(C / (VEC * CCH))), 256 threads.
template <typename T, int VEC>
static __global__ __launch_bounds__(256) void patch_sum_chan_kernel(PatchSumParams p, int CCH) {
  __shared__ float red[256 * VEC];
  const int tap = blockIdx.x, n = blockIdx.y;
  const int cc = threadIdx.x % CCH, ps = threadIdx.x / CCH, PS = 256 / CCH;
  const int c0 = (blockIdx.z * CCH + cc) * VEC;
  const int ky = tap / p.kw, kx = tap - ky * p.kw;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
  if (c0 < p.C && ps < PS) {
    const T* __restrict__ base = static_cast<const T*>(p.x) + static_cast<int64_t>(n) * p.sn + c0;
    int oy = ps / p.Wo, ox = ps - oy * p.Wo;
    const int adv_y = PS / p.Wo, adv_x = PS - adv_y * p.Wo;
    while (oy < p.Ho) {
      const int iy = oy * p.strh + ky - p.ph, ix = ox * p.strw + kx - p.pw;
      if (iy >= 0 && iy < p.H && ix >= 0 && ix < p.W) {
        const T* __restrict__ src = base + static_cast<int64_t>(iy) * p.sh + static_cast<int64_t>(ix) * p.sw;
        if constexpr (VEC == 8) {
          const uint4 raw = *reinterpret_cast<const uint4*>(src);       // 8 bf16
          const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[2 * e] += __builtin_bit_cast(float, w[e] << 16);
            acc[2 * e + 1] += __builtin_bit_cast(float, w[e] & 0xffff0000u);
          }
        } else {
          acc[0] += ps_load<T>(src);
        }
      }
      oy += adv_y;
      ox += adv_x;
      if (ox >= p.Wo) { ox -= p.Wo; ++oy; }
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) red[threadIdx.x * VEC + e] = acc[e];
  __syncthreads();
  if (ps == 0 && c0 < p.C) {
    for (int q = 1; q < PS; ++q) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] += red[(q * CCH + cc) * VEC + e];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if (c0 + e >= p.C) break;
      float* dst = p.out + static_cast<int64_t>(n) * p.ldo + static_cast<int64_t>(c0 + e) * (p.kh * p.kw) + tap;
      float v = p.alpha * acc[e];
      if (p.beta != 0.f) v += p.beta * *dst;
      *dst = v;
    }
  }
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
    // 16-byte loads of 8 bf16 channels when every pixel's channel run is 16-byte aligned
    const bool vec8 = dtype == AK_BF16 && C % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && sn % 8 == 0 &&
                      sh_el % 8 == 0 && sw_el % 8 == 0;
    const int64_t chunks = vec8 ? C / 8 : C;
    int cch = 1;
    while (cch < 256 && cch < chunks) cch *= 2;          // power of two <= 256 covering the chunks
    // few taps and samples (a 1 x 1 window at batch 64: 64 work groups): narrower channel ranges per work group, down
    // to 4 chunks = 64 contiguous bytes per position, until the grid fills the device
    while (cch > 4 && static_cast<int64_t>(kh) * kw * N * ((chunks + cch - 1) / cch) < 1024) cch /= 2;
    const int64_t zblocks = (chunks + cch - 1) / cch;
    if (zblocks > 65535 || N > 65535) return AK_ERR_UNSUPPORTED;
    dim3 grid(kh * kw, static_cast<unsigned>(N), static_cast<unsigned>(zblocks));
    if (vec8) hipLaunchKernelGGL((ak::patch_sum_chan_kernel<uint16_t, 8>), grid, dim3(256), 0, s, p, cch);
    else if (dtype == AK_BF16) hipLaunchKernelGGL((ak::patch_sum_chan_kernel<uint16_t, 1>), grid, dim3(256), 0, s, p, cch);
    else hipLaunchKernelGGL((ak::patch_sum_chan_kernel<float, 1>), grid, dim3(256), 0, s, p, cch);
  } else {
    if (C > 65535) return AK_ERR_UNSUPPORTED;
    dim3 grid(kh * kw, static_cast<unsigned>(C), static_cast<unsigned>(N));
    if (dtype == AK_BF16) hipLaunchKernelGGL(ak::patch_sum_col_kernel<uint16_t>, grid, dim3(64), 0, s, p);
    else hipLaunchKernelGGL(ak::patch_sum_col_kernel<float>, grid, dim3(64), 0, s, p);
  }
  return ak::check_launch();
}

namespace ak {
// lam_n[0] = n * lam[0]; ptrs[0] = gram, ptrs[1] = gram_inv: the device-side arguments of the batched Cholesky inverse
static __global__ void smw_setup_kernel(const float* __restrict__ lam, float n, float* __restrict__ lam_n,
                                        float** __restrict__ ptrs, float* gram, float* gram_inv) {
  if (threadIdx.x == 0) {
    lam_n[0] = n * lam[0];
    ptrs[0] = gram;
    ptrs[1] = gram_inv;
  }
}

static size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

struct SmwLayout {
  size_t gram, gram_inv, y, misc, chol, syrk, total;
};

static SmwLayout smw_layout(int64_t n, int64_t d) {
  SmwLayout l;
  size_t off = 0;
  l.gram = off; off += align256(static_cast<size_t>(n) * n * sizeof(float));
  l.gram_inv = off; off += align256(static_cast<size_t>(n) * n * sizeof(float));
  l.y = off; off += align256(static_cast<size_t>(n) * d * sizeof(float));
  l.misc = off; off += 256;                                   // lam_n, two pointers
  l.chol = off; off += align256(ak_chol_inv_ws_bytes(n, 1));
  l.syrk = off; off += align256(ak_conv_syrk_ws_bytes(1, n, 1, d, 1, 1, 1, 1, 0, 0));
  l.total = off;
  return l;
}
}  // namespace ak

extern "C" size_t ak_smw_inv_ws_bytes(int64_t n, int64_t d) {
  if (n <= 0 || d <= 0) return 0;
  return ak::smw_layout(n, d).total;
}

extern "C" int ak_smw_inv(const float* x, int64_t n, int64_t d, const float* lam, float* out, int64_t ldo, int* info,
                          void* ws, size_t ws_bytes, ak_stream_t stream) {
  if (x == nullptr || lam == nullptr || out == nullptr || info == nullptr || n <= 0 || d <= 0 || ldo < d)
    return AK_ERR_ARG;
  const ak::SmwLayout l = ak::smw_layout(n, d);
  if (ws == nullptr || ws_bytes < l.total || (reinterpret_cast<uintptr_t>(ws) & 255) != 0) return AK_ERR_WORKSPACE;
  char* base = static_cast<char*>(ws);
  float* gram = reinterpret_cast<float*>(base + l.gram);
  float* gram_inv = reinterpret_cast<float*>(base + l.gram_inv);
  float* y = reinterpret_cast<float*>(base + l.y);
  float* lam_n = reinterpret_cast<float*>(base + l.misc);
  float** ptrs = reinterpret_cast<float**>(base + l.misc + 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // gram = x x^T: the rows of x are the "channels" of a 1 x 1 convolution over d positions
  int rc = ak_conv_syrk(x, AK_F32, 1, n, 1, d, 1, 1, 1, 1, 0, 0, 1.f, 0.f, gram, n, base + l.syrk,
                        l.total - l.syrk, stream);
  if (rc != AK_OK) return rc;
  hipLaunchKernelGGL(ak::smw_setup_kernel, dim3(1), dim3(64), 0, s, lam, static_cast<float>(n), lam_n, ptrs, gram,
                     gram_inv);
  rc = ak_chol_inv_batched(ptrs, ptrs + 1, n, 1, lam_n, 1, nullptr, 0, info, base + l.chol, l.syrk - l.chol, stream);
  if (rc != AK_OK) return rc;
  rc = ak_gemm_f32(0, 0, n, d, n, 1.f, gram_inv, n, x, d, 0.f, y, d, 1, 0, 0, 0, stream);          // G^-1 x
  if (rc != AK_OK) return rc;
  rc = ak_gemm_f32(1, 0, d, d, n, 1.f, x, d, y, d, 0.f, out, ldo, 1, 0, 0, 0, stream);             // x^T G^-1 x
  if (rc != AK_OK) return rc;
  return ak_smw_finish(out, d, ldo, lam, stream);
}

extern "C" int ak_smw_finish(float* Z, int64_t d, int64_t ld, const float* lam, ak_stream_t stream) {
  if (Z == nullptr || lam == nullptr || d <= 0 || ld < d || d > 65535) return AK_ERR_ARG;
  dim3 grid(static_cast<unsigned>((d + 255) / 256), static_cast<unsigned>(d));
  hipLaunchKernelGGL(ak::smw_finish_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), Z, d, ld, lam);
  return ak::check_launch();
}
