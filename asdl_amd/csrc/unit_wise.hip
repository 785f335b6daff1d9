// Unit-wise (per feature 2x2) Fisher blocks of BatchNorm / LayerNorm, their damped inverses and the
// block-diagonal matrix-vector product.
//
// With the module output y, scale w and shift b, the normalised input is xh = (y - b_f) / w_f, and the
// per-sample gradients of feature f are  gw[n,f] = sum_s xh[n,f,s] * g[n,f,s],  gb[n,f] = sum_s g[n,f,s]
// (s runs over the spatial positions of BatchNorm2d; LayerNorm has a single position and one "sample" per row).
//   blocks[f] = beta * blocks[f] + alpha * sum_n [[gw^2, gw*gb], [gw*gb, gb^2]]
// Both tensors are read once, in whatever layout they have (strides in elements for sample, feature, position):
//   position-contiguous (NCHW): one wave per (sample, feature) reduces the positions;
//   feature-contiguous (NHWC, LayerNorm rows): threads run along the features, position lanes are reduced
//   through the LDS; with a single position the products are summed over a chunk of samples right away.
// A second pass sums over the samples (or chunks) in a fixed order.  Everything is fp32 arithmetic.
#include "common.hpp"

namespace ak {

struct UwParams {
  const void* y;
  const void* g;
  int y_bf16, g_bf16;
  const float* w;
  const float* b;
  int64_t N, F, S;
  int64_t ysn, ysf, yss, gsn, gsf, gss;
  float* part;          // [rows, F, 2] per-sample sums or [chunks, F, 3] product sums
  int64_t rows_per_chunk;
};

__device__ __forceinline__ float uw_load(const void* p, int is_bf16, int64_t idx) {
  if (is_bf16) {
    const uint32_t v = static_cast<uint32_t>(static_cast<const uint16_t*>(p)[idx]) << 16;
    return __builtin_bit_cast(float, v);
  }
  return static_cast<const float*>(p)[idx];
}

// position-contiguous: grid (F, N), one wave per (n, f)
static __global__ __launch_bounds__(64) void uw_rows_kernel(UwParams p) {
  const int64_t f = blockIdx.x, n = blockIdx.y;
  const float wf = p.w[f], bf = p.b[f];
  const int64_t yb = n * p.ysn + f * p.ysf, gb0 = n * p.gsn + f * p.gsf;
  float sw = 0.f, sb = 0.f;
  for (int64_t s = threadIdx.x; s < p.S; s += 64) {
    const float yv = uw_load(p.y, p.y_bf16, yb + s * p.yss);
    const float gv = uw_load(p.g, p.g_bf16, gb0 + s * p.gss);
    sw += (yv - bf) / wf * gv;
    sb += gv;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    sw += __shfl_xor(sw, o);
    sb += __shfl_xor(sb, o);
  }
  if (threadIdx.x == 0) {
    p.part[(n * p.F + f) * 2] = sw;
    p.part[(n * p.F + f) * 2 + 1] = sb;
  }
}

// feature-contiguous with several positions: grid (ceil(F/64), N), 256 threads = 64 features x 4 position lanes
static __global__ __launch_bounds__(256) void uw_cols_kernel(UwParams p) {
  __shared__ float red[2][4][64];
  const int fl = threadIdx.x & 63, sl = threadIdx.x >> 6;
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 64 + fl, n = blockIdx.y;
  float sw = 0.f, sb = 0.f;
  if (f < p.F) {
    const float wf = p.w[f], bf = p.b[f];
    const int64_t yb = n * p.ysn + f * p.ysf, gb0 = n * p.gsn + f * p.gsf;
    for (int64_t s = sl; s < p.S; s += 4) {
      const float yv = uw_load(p.y, p.y_bf16, yb + s * p.yss);
      const float gv = uw_load(p.g, p.g_bf16, gb0 + s * p.gss);
      sw += (yv - bf) / wf * gv;
      sb += gv;
    }
  }
  red[0][sl][fl] = sw;
  red[1][sl][fl] = sb;
  __syncthreads();
  if (sl == 0 && f < p.F) {
    p.part[(n * p.F + f) * 2] = red[0][0][fl] + red[0][1][fl] + red[0][2][fl] + red[0][3][fl];
    p.part[(n * p.F + f) * 2 + 1] = red[1][0][fl] + red[1][1][fl] + red[1][2][fl] + red[1][3][fl];
  }
}

// feature-contiguous, 16-byte loads: grid (ceil(F/FT), N, chunks of positions), 256 threads = 8 feature groups of VEC
// consecutive features x 32 position lanes.  part[((n * CH + ch) * F + f) * 2 + {0, 1}] = partial (gw, gb).
template <typename T>
static __global__ __launch_bounds__(256) void uw_cols_vec_kernel(UwParams p, int64_t pos_per_chunk) {
  constexpr int VEC = 16 / sizeof(T), FT = 8 * VEC;
  __shared__ float red[2][32][FT + 1];
  const int fg = threadIdx.x & 7, sl = threadIdx.x >> 3;
  const int64_t f0 = static_cast<int64_t>(blockIdx.x) * FT + fg * VEC, n = blockIdx.y, ch = blockIdx.z;
  const int64_t s_begin = ch * pos_per_chunk;
  const int64_t s_end = s_begin + pos_per_chunk < p.S ? s_begin + pos_per_chunk : p.S;
  float sw[VEC], sb[VEC], wf[VEC], bf[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) { sw[e] = sb[e] = 0.f; wf[e] = 1.f; bf[e] = 0.f; }
  const bool live = f0 < p.F;               // F is a multiple of VEC
  if (live) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) { wf[e] = 1.f / p.w[f0 + e]; bf[e] = p.b[f0 + e]; }
    const T* yp = static_cast<const T*>(p.y) + n * p.ysn + f0;
    const T* gp = static_cast<const T*>(p.g) + n * p.gsn + f0;
    for (int64_t s = s_begin + sl; s < s_end; s += 32) {
      const uint4 yv = *reinterpret_cast<const uint4*>(yp + s * p.yss);
      const uint4 gv = *reinterpret_cast<const uint4*>(gp + s * p.gss);
      const uint32_t yw[4] = {yv.x, yv.y, yv.z, yv.w}, gw4[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float ye, ge;
        if (sizeof(T) == 2) {
          const uint32_t ys = (e & 1) ? (yw[e >> 1] & 0xffff0000u) : (yw[e >> 1] << 16);
          const uint32_t gs = (e & 1) ? (gw4[e >> 1] & 0xffff0000u) : (gw4[e >> 1] << 16);
          ye = __builtin_bit_cast(float, ys);
          ge = __builtin_bit_cast(float, gs);
        } else {
          ye = __builtin_bit_cast(float, yw[e]);
          ge = __builtin_bit_cast(float, gw4[e]);
        }
        sw[e] += (ye - bf[e]) * wf[e] * ge;
        sb[e] += ge;
      }
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    red[0][sl][fg * VEC + e] = sw[e];
    red[1][sl][fg * VEC + e] = sb[e];
  }
  __syncthreads();
  if (threadIdx.x < 2 * FT) {
    const int which = threadIdx.x / FT, fl = threadIdx.x % FT;
    const int64_t f = static_cast<int64_t>(blockIdx.x) * FT + fl;
    if (f < p.F) {
      float acc = 0.f;
#pragma unroll
      for (int l = 0; l < 32; ++l) acc += red[which][l][fl];
      p.part[((n * gridDim.z + ch) * p.F + f) * 2 + which] = acc;
    }
  }
}

// feature-contiguous, one position (LayerNorm rows, BatchNorm1d): grid (ceil(F/256), chunks); the three product
// sums of a chunk of samples
static __global__ __launch_bounds__(256) void uw_cols_single_kernel(UwParams p) {
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (f >= p.F) return;
  const int64_t c = blockIdx.y;
  const int64_t n0 = c * p.rows_per_chunk;
  const int64_t n1 = n0 + p.rows_per_chunk < p.N ? n0 + p.rows_per_chunk : p.N;
  const float wf = p.w[f], bf = p.b[f];
  float ww = 0.f, wb = 0.f, bb = 0.f;
  for (int64_t n = n0; n < n1; ++n) {
    const float yv = uw_load(p.y, p.y_bf16, n * p.ysn + f * p.ysf);
    const float gv = uw_load(p.g, p.g_bf16, n * p.gsn + f * p.gsf);
    const float gw = (yv - bf) / wf * gv;
    ww += gw * gw;
    wb += gw * gv;
    bb += gv * gv;
  }
  float* dst = p.part + (c * p.F + f) * 3;
  dst[0] = ww; dst[1] = wb; dst[2] = bb;
}

// blocks[f] = beta*blocks[f] + alpha * sum over the partial rows; `width` 2: per-sample (gw, gb) in `chunks` pieces,
// 3: product sums.  grid ceil(F/64), 1024 threads = 64 features x 16 row lanes; fixed summation order.
static __global__ __launch_bounds__(1024) void uw_finalize_kernel(const float* __restrict__ part, int64_t rows, int64_t F,
                                                                  int width, int chunks, float alpha, float beta,
                                                                  float* __restrict__ blocks) {
  __shared__ float red[3][16][65];
  const int fl = threadIdx.x & 63, lane = threadIdx.x >> 6;
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 64 + fl;
  float ww = 0.f, wb = 0.f, bb = 0.f;
  if (f < F) {
    if (width == 2) {
      for (int64_t n = lane; n < rows; n += 16) {
        float gw = 0.f, gv = 0.f;
        for (int c = 0; c < chunks; ++c) {          // per-sample sums first: the positions were split over chunks
          gw += part[((n * chunks + c) * F + f) * 2];
          gv += part[((n * chunks + c) * F + f) * 2 + 1];
        }
        ww += gw * gw;
        wb += gw * gv;
        bb += gv * gv;
      }
    } else {
      for (int64_t n = lane; n < rows; n += 16) {
        ww += part[(n * F + f) * 3];
        wb += part[(n * F + f) * 3 + 1];
        bb += part[(n * F + f) * 3 + 2];
      }
    }
  }
  red[0][lane][fl] = ww;
  red[1][lane][fl] = wb;
  red[2][lane][fl] = bb;
  __syncthreads();
  if (lane == 0 && f < F) {
    ww = wb = bb = 0.f;
#pragma unroll
    for (int l = 0; l < 16; ++l) { ww += red[0][l][fl]; wb += red[1][l][fl]; bb += red[2][l][fl]; }
    float* dst = blocks + f * 4;
    float o0 = alpha * ww, o1 = alpha * wb, o3 = alpha * bb;
    if (beta != 0.f) { o0 += beta * dst[0]; o1 += beta * dst[1]; o3 += beta * dst[3]; }
    dst[0] = o0; dst[1] = o1; dst[2] = o1; dst[3] = o3;
  }
}

// inv[f] = (blocks[f] + damping I)^-1; info = 1-based index of the first singular block (0: none)
static __global__ __launch_bounds__(256) void uw_inv_kernel(const float* __restrict__ blocks, int64_t F, float damping,
                                                            float* __restrict__ inv, int* __restrict__ info) {
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (f >= F) return;
  const float a = blocks[f * 4] + damping, b = blocks[f * 4 + 1], c = blocks[f * 4 + 2], d = blocks[f * 4 + 3] + damping;
  const float det = a * d - b * c;
  if (det == 0.f || det != det) atomicMin(info, static_cast<int>(f) + 1);
  const float r = 1.f / det;
  inv[f * 4] = d * r;
  inv[f * 4 + 1] = -b * r;
  inv[f * 4 + 2] = -c * r;
  inv[f * 4 + 3] = a * r;
}

// all-zero test of the blocks: flag[0] = 1 when any entry is non-zero; also resets info for the inverse
static __global__ __launch_bounds__(256) void uw_nonzero_kernel(const float* __restrict__ blocks, int64_t n, int* flag) {
  int any = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
    any |= (blocks[i] != 0.f);
  if (__syncthreads_or(any) && threadIdx.x == 0) flag[0] = 1;
}

// uw_nonzero_kernel + uw_inv_kernel for many modules in one launch.  `table`: one row of 6 int64 per module: blocks,
// inv, flags (addresses; flags = int[2] preset to {0, 0x7fffffff}), F, first block (blocks of 256 features, running
// sum), damping (float bits).
static __global__ __launch_bounds__(256) void uw_inv_grouped_kernel(const int64_t* __restrict__ table, int count) {
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * 6 + 4] <= w) lo = mid;
    else hi = mid - 1;
  }
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * 6;
  const float* __restrict__ blocks = reinterpret_cast<const float*>(r[0]);
  float* __restrict__ inv = reinterpret_cast<float*>(r[1]);
  int* flags = reinterpret_cast<int*>(r[2]);
  const int64_t F = r[3];
  const float damping = __builtin_bit_cast(float, static_cast<uint32_t>(r[5]));
  const int64_t f = static_cast<int64_t>(w - r[4]) * 256 + threadIdx.x;
  int any = 0;
  if (f < F) {
    const float b0 = blocks[f * 4], b1 = blocks[f * 4 + 1], b2 = blocks[f * 4 + 2], b3 = blocks[f * 4 + 3];
    any = (b0 != 0.f) | (b1 != 0.f) | (b2 != 0.f) | (b3 != 0.f);
    const float a = b0 + damping, d = b3 + damping;
    const float det = a * d - b1 * b2;
    if (det == 0.f || det != det) atomicMin(flags + 1, static_cast<int>(f) + 1);
    const float q = 1.f / det;
    inv[f * 4] = d * q;
    inv[f * 4 + 1] = -b1 * q;
    inv[f * 4 + 2] = -b2 * q;
    inv[f * 4 + 3] = a * q;
  }
  if (__syncthreads_or(any) && threadIdx.x == 0) flags[0] = 1;
}

static __global__ void uw_reset_kernel(int* flag, int* info) {
  flag[0] = 0;
  info[0] = 0x7fffffff;
}

static __global__ __launch_bounds__(256) void uw_mvp_kernel(const float* __restrict__ mat, int64_t F, float* __restrict__ vw,
                                                            float* __restrict__ vb, float scale) {
  const int64_t f = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (f >= F) return;
  const float w = vw[f] * scale, b = vb[f] * scale;
  vw[f] = mat[f * 4] * w + mat[f * 4 + 1] * b;
  vb[f] = mat[f * 4 + 2] * w + mat[f * 4 + 3] * b;
}

// The same for many modules in one launch.  `table`: one row of 5 int64 per module: blocks, vec_weight, vec_bias
// (addresses), F, first block (blocks of 256 features, running sum).
static __global__ __launch_bounds__(256) void uw_mvp_grouped_kernel(const int64_t* __restrict__ table, int count,
                                                                    float scale) {
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * 5 + 4] <= w) lo = mid;
    else hi = mid - 1;
  }
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * 5;
  const float* __restrict__ mat = reinterpret_cast<const float*>(r[0]);
  float* __restrict__ vw = reinterpret_cast<float*>(r[1]);
  float* __restrict__ vb = reinterpret_cast<float*>(r[2]);
  const int64_t f = static_cast<int64_t>(w - r[4]) * 256 + threadIdx.x;
  if (f >= r[3]) return;
  const float wv = vw[f] * scale, bv = vb[f] * scale;
  vw[f] = mat[f * 4] * wv + mat[f * 4 + 1] * bv;
  vb[f] = mat[f * 4 + 2] * wv + mat[f * 4 + 3] * bv;
}

constexpr int64_t kUwChunkRows = 64;

// Chunks of positions per (sample, feature tile) for the vector kernel: enough work groups to fill the device.
static int uw_chunks(int64_t N, int64_t F, int64_t S, int ft) {
  const int64_t tiles = N * ((F + ft - 1) / ft);
  int64_t ch = (2048 + tiles - 1) / tiles;
  const int64_t max_ch = (S + 127) / 128;         // at least 128 positions per chunk
  if (ch > max_ch) ch = max_ch;
  if (ch < 1) ch = 1;
  if (ch > 64) ch = 64;
  return static_cast<int>(ch);
}

}  // namespace ak

extern "C" size_t ak_unit_wise_ws_bytes(int64_t N, int64_t F, int64_t S) {
  if (N <= 0 || F <= 0 || S <= 0) return 0;
  if (S == 1) return static_cast<size_t>((N + ak::kUwChunkRows - 1) / ak::kUwChunkRows) * F * 3 * sizeof(float);
  return static_cast<size_t>(N) * F * 2 * sizeof(float) * ak::uw_chunks(N, F, S, 32);    // upper bound over both layouts
}

extern "C" int ak_unit_wise_stats(const void* y, int y_dtype, int64_t ysn, int64_t ysf, int64_t yss, const void* g,
                                  int g_dtype, int64_t gsn, int64_t gsf, int64_t gss, const float* weight,
                                  const float* bias, int64_t N, int64_t F, int64_t S, float alpha, float beta,
                                  float* blocks, void* ws, size_t ws_bytes, ak_stream_t stream) {
  using namespace ak;
  if (y == nullptr || g == nullptr || weight == nullptr || bias == nullptr || blocks == nullptr || N <= 0 || F <= 0 ||
      S <= 0)
    return AK_ERR_ARG;
  if ((y_dtype != AK_F32 && y_dtype != AK_BF16) || (g_dtype != AK_F32 && g_dtype != AK_BF16)) return AK_ERR_ARG;
  if (N > 65535 && S > 1) return AK_ERR_UNSUPPORTED;            // grid.y
  if (ws == nullptr || ws_bytes < ak_unit_wise_ws_bytes(N, F, S)) return AK_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  UwParams p;
  p.y = y; p.g = g; p.y_bf16 = y_dtype == AK_BF16; p.g_bf16 = g_dtype == AK_BF16;
  p.w = weight; p.b = bias; p.N = N; p.F = F; p.S = S;
  p.ysn = ysn; p.ysf = ysf; p.yss = yss; p.gsn = gsn; p.gsf = gsf; p.gss = gss;
  p.part = static_cast<float*>(ws);
  p.rows_per_chunk = kUwChunkRows;
  int64_t rows;
  int width, chunks = 1;
  if (S == 1) {
    rows = (N + kUwChunkRows - 1) / kUwChunkRows;
    width = 3;
    if (rows > 65535) return AK_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(uw_cols_single_kernel, dim3(static_cast<unsigned>((F + 255) / 256), static_cast<unsigned>(rows)),
                       dim3(256), 0, s, p);
  } else {
    rows = N;
    width = 2;
    const int vec = y_dtype == AK_BF16 ? 8 : 4;
    const bool vec_ok = ysf == 1 && gsf == 1 && y_dtype == g_dtype && F % vec == 0 && ysn % vec == 0 && gsn % vec == 0 &&
                        yss % vec == 0 && gss % vec == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
                        (reinterpret_cast<uintptr_t>(g) & 15) == 0;
    if (yss == 1 && gss == 1) {
      if (F > 0x7fffffff) return AK_ERR_UNSUPPORTED;
      hipLaunchKernelGGL(uw_rows_kernel, dim3(static_cast<unsigned>(F), static_cast<unsigned>(N)), dim3(64), 0, s, p);
    } else if (vec_ok) {
      const int ft = 8 * vec;
      chunks = uw_chunks(N, F, S, ft);
      const int64_t per = (S + chunks - 1) / chunks;
      dim3 grid(static_cast<unsigned>((F + ft - 1) / ft), static_cast<unsigned>(N), static_cast<unsigned>(chunks));
      if (y_dtype == AK_BF16) hipLaunchKernelGGL(uw_cols_vec_kernel<uint16_t>, grid, dim3(256), 0, s, p, per);
      else hipLaunchKernelGGL(uw_cols_vec_kernel<float>, grid, dim3(256), 0, s, p, per);
    } else {
      hipLaunchKernelGGL(uw_cols_kernel, dim3(static_cast<unsigned>((F + 63) / 64), static_cast<unsigned>(N)), dim3(256),
                         0, s, p);
    }
  }
  hipLaunchKernelGGL(uw_finalize_kernel, dim3(static_cast<unsigned>((F + 63) / 64)), dim3(1024), 0, s, p.part, rows, F,
                     width, chunks, alpha, beta, blocks);
  return check_launch();
}

extern "C" int ak_unit_wise_inv(const float* blocks, int64_t F, float damping, float* inv, int* flags,
                                ak_stream_t stream) {
  using namespace ak;
  if (blocks == nullptr || inv == nullptr || flags == nullptr || F <= 0) return AK_ERR_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(uw_reset_kernel, dim3(1), dim3(1), 0, s, flags, flags + 1);
  int64_t scan_blocks = (4 * F + 255) / 256;
  if (scan_blocks > 1024) scan_blocks = 1024;
  hipLaunchKernelGGL(uw_nonzero_kernel, dim3(static_cast<unsigned>(scan_blocks)), dim3(256), 0, s, blocks, 4 * F, flags);
  hipLaunchKernelGGL(uw_inv_kernel, dim3(static_cast<unsigned>((F + 255) / 256)), dim3(256), 0, s, blocks, F, damping, inv,
                     flags + 1);
  return check_launch();
}

extern "C" int ak_unit_wise_mvp(const float* mat, int64_t F, float* vec_weight, float* vec_bias, float scale,
                                ak_stream_t stream) {
  using namespace ak;
  if (mat == nullptr || vec_weight == nullptr || vec_bias == nullptr || F <= 0) return AK_ERR_ARG;
  hipLaunchKernelGGL(uw_mvp_kernel, dim3(static_cast<unsigned>((F + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), mat, F, vec_weight, vec_bias, scale);
  return check_launch();
}

extern "C" int ak_unit_wise_mvp_grouped(const int64_t* table, int count, int64_t total_blocks, float scale,
                                        ak_stream_t stream) {
  using namespace ak;
  if (count < 0 || total_blocks < 0 || total_blocks > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_blocks == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipLaunchKernelGGL(uw_mvp_grouped_kernel, dim3(static_cast<unsigned>(total_blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), table, count, scale);
  return check_launch();
}

extern "C" int ak_unit_wise_inv_grouped(const int64_t* table, int count, int64_t total_blocks, ak_stream_t stream) {
  using namespace ak;
  if (count < 0 || total_blocks < 0 || total_blocks > (1ll << 30)) return AK_ERR_ARG;
  if (count == 0 || total_blocks == 0) return AK_OK;
  if (table == nullptr) return AK_ERR_ARG;
  hipLaunchKernelGGL(uw_inv_grouped_kernel, dim3(static_cast<unsigned>(total_blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), table, count);
  return check_launch();
}
