// Shampoo's inverse p-th root of a batch of same-size symmetric PSD statistics:
//   out <- (S + r I)^(-1/p),  r = ridge_eps * lambda_max(S),
// power iteration for lambda_max followed by the coupled Newton iteration, with every convergence
// test evaluated on the device.  The host enqueues the maximum number of iterations; each kernel
// first reads its matrix's `active` word and returns at once when that matrix has converged (or
// stopped because its error grew by more than 1.2x, in which case the previous root is kept).
// Statistics of 512 columns and more keep every matrix of the iteration as 16-bit planes and multiply them with the
// plane kernel (gemm_planes.hpp); smaller ones keep fp32 matrices and run on the split-operand tile kernel (gemm_x3.hpp)
// or the fp32 tile of gemm_f32.hpp.  All sum in chunks; the product that forms the next M also folds max |M - I| into a
// device word and writes the next step's polynomial, and the iterates alternate between two buffer pairs, so a step is
// its products and one decision kernel.
#include <cmath>
#include <cstdlib>
#include "gemm_f32.hpp"
#include "gemm_planes.hpp"

namespace ak {

// products of the Newton iteration: 3 = split-bf16 kernel (fp32-grade accuracy), 0 = fp32 MFMA
#ifdef AK_TUNING_HOOKS
inline int g_root_split = 3;
#else
constexpr int g_root_split = 3;
#endif

constexpr int RCHUNKS = 64;   // partial-reduction chunks per matrix
constexpr int kRootSymmetricMinDim = 512;   // products of matrices this large compute the lower tiles only
// Statistics this large iterate on bf16 planes (gemm_planes.hpp): every matrix of the iteration is stored as the three
// planes of its exact split, written by the product that makes it.  Smaller ones keep fp32 matrices and the tile
// kernels that split (or multiply in fp32) as they read.
#ifdef AK_TUNING_HOOKS
inline int g_root_planes_min = 512;
#else
constexpr int g_root_planes_min = 512;
#endif
static bool root_uses_planes(int64_t n) { return n >= g_root_planes_min && n <= kPlaneMaxDim; }

// Scales of the two-plane fp16 form (gemm_planes.hpp).  M, the polynomials T and their powers are bounded by the
// normalisation of the iteration: ||M_0||_F = (1 + p) / 2, T <= (1 + 1/p) I and T^k <= e for a positive definite
// statistic, so 2^12 keeps them (and a fair excess of an indefinite input) below the fp16 maximum.  The root is kept
// without its factor z^(1/p): it grows from I to (z A)^(-1/p) <= lambda_min(M_0)^(-1/p), and the ridge bounds
// lambda_min(M_0) >= ridge_eps (1 + p) / (2 sqrt(n)) from below (lambda_max from the power iteration; a value that is
// low by a factor f moves the bound by f^(1/p), which the four spare bits cover).  The root's scale must not be below
// one (the identity it starts from needs its 22 bits too), so the bound has to stay below 2^12: p = 4 with a ridge
// of 1e-6 gives 70, p = 2 at the same ridge 8000 and more.  Beyond that, without a ridge, or with a power above 8 the
// iteration stays on the bf16 planes, which have the range of fp32.
constexpr float kRootScaleM = 4096.f;
static bool root_fp16_allowed() {
  static const bool on = [] {
    const char* e = std::getenv("ASDL_AMD_ROOT_FP16_PLANES");
    return e == nullptr || e[0] != '0';
  }();
  return on;
}
// 0: not on fp16 planes; else the scale of the root's planes
static float root_fp16_scale(int64_t n, int p, float ridge_eps) {
  if (!root_fp16_allowed() || !root_uses_planes(n) || p > 8 || !(ridge_eps > 0.f)) return 0.f;
  const double lam = static_cast<double>(ridge_eps) * (1 + p) / (2.0 * std::sqrt(static_cast<double>(n)));
  const double bound = std::pow(lam, -1.0 / p);                 // of the root's largest eigenvalue
  if (!(bound < 1e30)) return 0.f;
  const int e = 12 - static_cast<int>(std::ceil(std::log2(bound)));
  if (e < 0) return 0.f;
  return static_cast<float>(std::ldexp(1.0, e < 12 ? e : 12));
}
static int64_t root_pad(int64_t n) { return (n + kPlaneTile - 1) / kPlaneTile * kPlaneTile; }
// floats of the matrix buffers of one statistic: ten plane sets (two roots, two M, two T, four products) of
// 3 n_pad^2 bf16, or nine fp32 matrices (two M, the second root, two T, four products)
static size_t root_matrix_floats(int64_t n) {
  if (root_uses_planes(n)) return static_cast<size_t>(15) * root_pad(n) * root_pad(n);
  return static_cast<size_t>(9) * n * n;
}

struct RootState {
  // per matrix, all device memory
  float* sv;        // current eigenvalue estimate
  float* nrm2;      // squared norm of the current power-iteration vector
  float* err;       // current Newton error max|M - I|
  float* zscale;
  float* partial;   // [batch, RCHUNKS]
  int* pi_active;   // power iteration still running
  int* pi_iters;
  int* active;      // Newton iteration still running
  int* commit;      // last Newton step accepted
  int* count;
  int* par;         // which of the two root / M buffers holds the matrix's latest accepted iterate
  float* errword;   // max |M' - I| of the step under way, folded in by the epilogue of the product that forms M'
  int* ovf;         // fp16 planes: a product of the step under way left the fp16 range
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

// grid (batch): v <- v0, norm, flags
static __global__ __launch_bounds__(256) void root_init_kernel(RootState st, const float* __restrict__ v0,
                                                               float* __restrict__ v, int64_t n) {
  __shared__ float red[4];
  const int z = blockIdx.x;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 256) {
    const float x = v0[z * n + i];
    v[z * n + i] = x;
    s += x * x;
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    st.nrm2[z] = red[0] + red[1] + red[2] + red[3];
    st.sv[z] = 0.f;
    st.pi_active[z] = 1;
    st.pi_iters[z] = 0;
    st.active[z] = 0;
    st.commit[z] = 0;
    st.count[z] = 0;
    st.par[z] = 0;
    st.errword[z] = 0.f;
    st.ovf[z] = 0;
  }
}

// grid (ceil(n/4), batch): mv[row] = S[row,:] . v / ||v||   (one wave per row)
static __global__ __launch_bounds__(256) void power_matvec_kernel(RootState st, const float* __restrict__ S,
                                                                  int64_t strideS, const float* __restrict__ v,
                                                                  float* __restrict__ mv, int64_t n) {
  const int z = blockIdx.y;
  if (st.pi_active[z] == 0) return;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= n) return;
  const int lane = threadIdx.x & 63;
  const float* __restrict__ Sr = S + z * strideS + row * n;
  const float* __restrict__ vz = v + z * n;
  float s = 0.f;
  for (int64_t k = lane; k < n; k += 64) s += Sr[k] * vz[k];
  s = wave_sum(s);
  if (lane == 0) mv[z * n + row] = s / sqrtf(st.nrm2[z]);
}

// grid (batch): s_v = (v/||v||) . mv; error = |s_v - sv|; v <- mv
static __global__ __launch_bounds__(256) void power_update_kernel(RootState st, float* __restrict__ v,
                                                                  const float* __restrict__ mv, int64_t n, float tol,
                                                                  int max_iters) {
  __shared__ float red[8];
  const int z = blockIdx.x;
  if (st.pi_active[z] == 0) return;
  const float inv_norm = 1.f / sqrtf(st.nrm2[z]);
  float dot = 0.f, nn = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 256) {
    const float m = mv[z * n + i];
    dot += v[z * n + i] * inv_norm * m;
    nn += m * m;
    v[z * n + i] = m;
  }
  dot = wave_sum(dot);
  nn = wave_sum(nn);
  if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = dot; red[4 + (threadIdx.x >> 6)] = nn; }
  __syncthreads();
  if (threadIdx.x == 0) {
    const float s_v = red[0] + red[1] + red[2] + red[3];
    const float error = fabsf(s_v - st.sv[z]);
    st.sv[z] = s_v;
    st.nrm2[z] = red[4] + red[5] + red[6] + red[7];
    const int it = st.pi_iters[z] + 1;
    st.pi_iters[z] = it;
    if (!(error > tol && it < max_iters)) st.pi_active[z] = 0;
  }
}

// grid (RCHUNKS, batch): S += ridge I (in place), partial sum of squares of the ridged matrix
static __global__ __launch_bounds__(256) void root_ridge_kernel(RootState st, float* __restrict__ S, int64_t strideS,
                                                                int64_t n, float ridge_eps) {
  __shared__ float red[4];
  const int z = blockIdx.y;
  float* __restrict__ Sz = S + z * strideS;
  const float ridge = ridge_eps * st.sv[z];
  const int64_t total = n * n;
  float s = 0.f;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += RCHUNKS * 256) {
    float x = Sz[i];
    if (i % (n + 1) == 0) {
      x += ridge;
      Sz[i] = x;
    }
    s += x * x;
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) st.partial[z * RCHUNKS + blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

// grid (batch)
static __global__ void root_zscale_kernel(RootState st, int p) {
  const int z = blockIdx.x;
  if (threadIdx.x != 0) return;
  float s = 0.f;
  for (int c = 0; c < RCHUNKS; ++c) s += st.partial[z * RCHUNKS + c];
  st.zscale[z] = (1.f + p) / (2.f * sqrtf(s));
}

// grid (RCHUNKS, batch): M = z S, T = (1 + 1/p) I - M / p, root = z^(1/p) I, partial max |M - I|
static __global__ __launch_bounds__(256) void root_start_kernel(RootState st, const float* __restrict__ S,
                                                                int64_t strideS, float* __restrict__ M,
                                                                float* __restrict__ T, float* __restrict__ root,
                                                                int64_t strideR, int64_t n, int p) {
  __shared__ float red[4];
  const int z = blockIdx.y;
  const float zs = st.zscale[z];
  const float r0 = powf(zs, 1.0f / p);
  const float alpha = -1.0f / p;
  const int64_t total = n * n;
  float e = 0.f;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += RCHUNKS * 256) {
    const bool diag = (i % (n + 1) == 0);
    const float m = zs * S[z * strideS + i];
    M[z * total + i] = m;
    T[z * total + i] = (diag ? (1.f - alpha) : 0.f) + alpha * m;
    root[z * strideR + i] = diag ? r0 : 0.f;
    e = fmaxf(e, fabsf(m - (diag ? 1.f : 0.f)));
  }
  e = wave_max(e);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = e;
  __syncthreads();
  if (threadIdx.x == 0) st.partial[z * RCHUNKS + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// grid (batch)
static __global__ void root_begin_kernel(RootState st, float tol, int max_iter) {
  const int z = blockIdx.x;
  if (threadIdx.x != 0) return;
  float e = 0.f;
  for (int c = 0; c < RCHUNKS; ++c) e = fmaxf(e, st.partial[z * RCHUNKS + c]);
  st.err[z] = e;
  st.active[z] = (e > tol && max_iter > 0) ? 1 : 0;
}

// grid (batch): accept / reject the step and decide whether to go on.  The error of the step is the word the product
// M' = T^p M folded max |M' - I| into; `wrote`: which buffer pair that step wrote (the matrix's latest iterate if
// the step is accepted).
static __global__ void newton_decide_kernel(RootState st, float tol, int max_iter, int wrote) {
  const int z = blockIdx.x;
  if (threadIdx.x != 0) return;
  st.commit[z] = 0;
  const float e = st.errword[z];
  st.errword[z] = 0.f;
  const int overflow = st.ovf[z];
  st.ovf[z] = 0;
  if (st.active[z] == 0) return;
  const float err = st.err[z];
  // diverging: keep the previous root (NaN compares false, like the reference).  A step whose products left the range
  // of the fp16 planes (a statistic far from positive definite) is dropped the same way.
  if (overflow != 0 || e > err * 1.2f) {
    st.active[z] = 0;
    return;
  }
  st.commit[z] = 1;
  st.par[z] = wrote;
  st.err[z] = e;
  const int c = st.count[z] + 1;
  st.count[z] = c;
  if (!(e > tol && c < max_iter)) st.active[z] = 0;
}

// grid (RCHUNKS, batch): brings the matrices whose latest iterate sits in the second buffer pair back to the first
// one (root, M, and T for a matrix that goes on iterating) and resets their marks.  With an even number of iterations
// per call only the matrices that stopped after an odd number of steps are concerned.
static __global__ __launch_bounds__(256) void newton_gather_kernel(RootState st, float* __restrict__ root,
                                                                   int64_t strideR, const float* __restrict__ root1,
                                                                   float* __restrict__ M, const float* __restrict__ M1,
                                                                   float* __restrict__ T, const float* __restrict__ T1,
                                                                   int64_t n) {
  const int z = blockIdx.y;
  if (st.par[z] == 0) return;
  const bool go_on = st.active[z] != 0;
  const int64_t total = n * n;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += RCHUNKS * 256) {
    root[z * strideR + i] = root1[z * total + i];
    M[z * total + i] = M1[z * total + i];
    if (go_on) T[z * total + i] = T1[z * total + i];
  }
}

// grid (batch): after newton_gather_kernel
static __global__ void newton_gathered_kernel(RootState st) {
  if (threadIdx.x == 0) st.par[blockIdx.x] = 0;
}

// ---- the same on bf16 planes --------------------------------------------------------------------------------------

// grid (RCHUNKS, batch): planes of M = z S, T = (1 + 1/p) I - M / p and root = z^(1/p) I over the padded index range
// (zero outside n x n), partial max |M - I|.  NP = 2 (fp16 planes): M and T scaled by scale_m, the root without its
// factor z^(1/p): scale_r I.
template <int NP>
static __global__ __launch_bounds__(256) void root_start_planes_kernel(RootState st, const float* __restrict__ S,
                                                                       int64_t strideS, __bf16* __restrict__ M,
                                                                       __bf16* __restrict__ T, __bf16* __restrict__ R,
                                                                       int64_t set_elems, int64_t n, int64_t n_pad, int p,
                                                                       float scale_m, float scale_r) {
  __shared__ float red[4];
  const int z = blockIdx.y;
  const float zs = st.zscale[z];
  const float r0 = NP == 2 ? scale_r : powf(zs, 1.0f / p);
  const float sm = NP == 2 ? scale_m : 1.f;
  const float alpha = -1.0f / p;
  const int64_t total = n_pad * n_pad;
  unsigned short* Mz = reinterpret_cast<unsigned short*>(M) + z * set_elems;
  unsigned short* Tz = reinterpret_cast<unsigned short*>(T) + z * set_elems;
  unsigned short* Rz = reinterpret_cast<unsigned short*>(R) + z * set_elems;
  float e = 0.f;
  for (int64_t at = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; at < total; at += RCHUNKS * 256) {
    const int64_t i = at / n_pad, j = at - i * n_pad;
    const bool inside = i < n && j < n, diag = i == j;
    float m = 0.f, t = 0.f, r = 0.f;
    if (inside) {
      m = zs * S[z * strideS + i * n + j];
      t = (diag ? (1.f - alpha) : 0.f) + alpha * m;
      r = diag ? r0 : 0.f;
      e = fmaxf(e, fabsf(m - (diag ? 1.f : 0.f)));
    }
    unsigned short o[3];
    const int64_t dst = plane_index(i, j, n_pad);
    plane_bits<NP>(m * sm, o);
#pragma unroll
    for (int q = 0; q < NP; ++q) Mz[q * total + dst] = o[q];
    plane_bits<NP>(t * sm, o);
#pragma unroll
    for (int q = 0; q < NP; ++q) Tz[q * total + dst] = o[q];
    plane_bits<NP>(r, o);
#pragma unroll
    for (int q = 0; q < NP; ++q) Rz[q * total + dst] = o[q];
  }
  e = wave_max(e);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = e;
  __syncthreads();
  if (threadIdx.x == 0) st.partial[z * RCHUNKS + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

// grid (RCHUNKS, batch): newton_gather_kernel on plane sets (set_words 32-bit words each)
static __global__ __launch_bounds__(256) void newton_gather_planes_kernel(RootState st, uint32_t* __restrict__ R0,
                                                                          const uint32_t* __restrict__ R1,
                                                                          uint32_t* __restrict__ M0,
                                                                          const uint32_t* __restrict__ M1,
                                                                          uint32_t* __restrict__ T0,
                                                                          const uint32_t* __restrict__ T1,
                                                                          int64_t set_words) {
  const int z = blockIdx.y;
  if (st.par[z] == 0) return;
  const bool go_on = st.active[z] != 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < set_words; i += RCHUNKS * 256) {
    R0[z * set_words + i] = R1[z * set_words + i];
    M0[z * set_words + i] = M1[z * set_words + i];
    if (go_on) T0[z * set_words + i] = T1[z * set_words + i];
  }
}

// grid (RCHUNKS, batch): the caller's fp32 result from the planes of the root (their sum is exact).  NP = 2: the planes
// hold scale_r times the root without its factor z^(1/p); zscale == nullptr: no such factor (plain product).
template <int NP>
static __global__ __launch_bounds__(256) void root_out_planes_kernel(const __bf16* __restrict__ R, int64_t set_elems,
                                                                     float* __restrict__ out, int64_t strideOut,
                                                                     int64_t n, int64_t n_pad, const float* zscale, int p,
                                                                     float scale_r) {
  const int z = blockIdx.y;
  const int64_t total = n_pad * n_pad;
  if constexpr (NP == 3) {
    const __bf16* Rz = R + z * set_elems;
    for (int64_t at = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; at < n * n; at += RCHUNKS * 256) {
      const int64_t i = at / n, j = at - i * n;
      const int64_t src = plane_index(i, j, n_pad);
      out[z * strideOut + at] = (static_cast<float>(Rz[src]) + static_cast<float>(Rz[total + src])) +
                                static_cast<float>(Rz[2 * total + src]);
    }
  } else {
    const _Float16* Rz = reinterpret_cast<const _Float16*>(R) + z * set_elems;
    const float mul = (zscale != nullptr ? powf(zscale[z], 1.0f / p) : 1.f) / scale_r;
    for (int64_t at = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; at < n * n; at += RCHUNKS * 256) {
      const int64_t i = at / n, j = at - i * n;
      const int64_t src = plane_index(i, j, n_pad);
      out[z * strideOut + at] = mul * (static_cast<float>(Rz[src]) + static_cast<float>(Rz[total + src]));
    }
  }
}

// grid (batch)
static __global__ void root_stats_kernel(RootState st, float* __restrict__ stats) {
  const int z = blockIdx.x;
  if (threadIdx.x != 0) return;
  stats[4 * z] = st.sv[z];
  stats[4 * z + 1] = static_cast<float>(st.pi_iters[z]);
  stats[4 * z + 2] = static_cast<float>(st.count[z]);
  stats[4 * z + 3] = st.err[z];
}

static size_t root_state_floats(int batch) { return static_cast<size_t>(batch) * (4 + RCHUNKS + 8) + 16; }

}  // namespace ak

extern "C" size_t ak_inv_root_ws_bytes(int64_t n, int batch) {
  if (n <= 0 || batch <= 0) return 0;
  // the matrix buffers, two vectors, state
  return (static_cast<size_t>(batch) * (ak::root_matrix_floats(n) + 2 * n) + ak::root_state_floats(batch)) * sizeof(float);
}

namespace ak {

// Workspace layout: M (two buffers), the second root buffer (the first is the caller's result), T (two buffers), four
// product buffers, two vectors, then the per-matrix state; `active` (int32 per matrix, non-zero while its Newton
// iteration runs) sits at root_active_offset().
static size_t root_active_offset(int64_t n, int batch) {
  return (static_cast<size_t>(batch) * (root_matrix_floats(n) + 2 * n) + static_cast<size_t>(batch) * (4 + RCHUNKS + 2)) * sizeof(float);
}

// phases: 1 = power iteration, ridge and start of the Newton iteration; 2 = `iters` Newton iterations; 4 = statistics
static int inv_root_run(int phases, int iters, float* S, int64_t n, int batch, int64_t strideS, int p, float ridge_eps,
                        const float* v0, int max_power_iter, float power_tol, int max_iter, float tol, float* out,
                        int64_t strideOut, float* stats, void* ws, size_t ws_bytes, ak_stream_t stream) {
  if (S == nullptr || v0 == nullptr || out == nullptr || stats == nullptr || n < 2 || batch <= 0 || p < 1 ||
      n > (1 << 20) || strideS < n * n || strideOut < n * n)
    return AK_ERR_ARG;
  if (ws == nullptr || ws_bytes < ak_inv_root_ws_bytes(n, batch)) return AK_ERR_WORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t nn = n * n;
  float* w = static_cast<float*>(ws);
  const bool planes = root_uses_planes(n);
  // two fp16 planes where the ridge bounds the root, else three bf16 planes; every part of a computation in parts
  // gets the same ridge_eps and p, hence the same answer
  const float scale_r = root_fp16_scale(n, p, ridge_eps);
  const int np = scale_r > 0.f ? 2 : 3;
  const int64_t n_pad = root_pad(n), set_elems = np * n_pad * n_pad;      // 16-bit elements of one plane set
  float* Mb[2] = {nullptr, nullptr};
  float* root1 = nullptr;
  float* Tb[2] = {nullptr, nullptr};
  float* buf[4] = {nullptr, nullptr, nullptr, nullptr};
  __bf16* pR[2] = {nullptr, nullptr};
  __bf16* pM[2] = {nullptr, nullptr};
  __bf16* pT[2] = {nullptr, nullptr};
  __bf16* pbuf[4] = {nullptr, nullptr, nullptr, nullptr};
  if (planes) {
    __bf16* q = reinterpret_cast<__bf16*>(w);
    for (int i = 0; i < 2; ++i) { pR[i] = q; q += batch * set_elems; }
    for (int i = 0; i < 2; ++i) { pM[i] = q; q += batch * set_elems; }
    for (int i = 0; i < 2; ++i) { pT[i] = q; q += batch * set_elems; }
    for (int i = 0; i < 4; ++i) { pbuf[i] = q; q += batch * set_elems; }
  } else {
    float* q = w;
    Mb[0] = q;           q += batch * nn;
    Mb[1] = q;           q += batch * nn;
    root1 = q;           q += batch * nn;
    Tb[0] = q;           q += batch * nn;
    Tb[1] = q;           q += batch * nn;
    for (int i = 0; i < 4; ++i) { buf[i] = q; q += batch * nn; }
  }
  w += static_cast<size_t>(batch) * root_matrix_floats(n);
  float* v = w;        w += batch * n;
  float* mv = w;       w += batch * n;
  RootState st;
  st.sv = w; w += batch;
  st.nrm2 = w; w += batch;
  st.err = w; w += batch;
  st.zscale = w; w += batch;
  st.partial = w; w += static_cast<size_t>(batch) * RCHUNKS;
  st.pi_active = reinterpret_cast<int*>(w); w += batch;
  st.pi_iters = reinterpret_cast<int*>(w); w += batch;
  st.active = reinterpret_cast<int*>(w); w += batch;
  st.commit = reinterpret_cast<int*>(w); w += batch;
  st.count = reinterpret_cast<int*>(w); w += batch;
  st.par = reinterpret_cast<int*>(w); w += batch;
  st.errword = w; w += batch;
  st.ovf = reinterpret_cast<int*>(w); w += batch;

  if (reinterpret_cast<unsigned char*>(st.active) != static_cast<unsigned char*>(ws) + root_active_offset(n, batch))
    return AK_ERR_ARG;     // the layout above and root_active_offset() have to agree
  const dim3 gb(batch), gc(RCHUNKS, batch), b256(256);
  if (phases & 1) {
    hipLaunchKernelGGL(root_init_kernel, gb, b256, 0, s, st, v0, v, n);
    const dim3 gmv(static_cast<unsigned>((n + 3) / 4), batch);
    for (int it = 0; it < max_power_iter; ++it) {
      hipLaunchKernelGGL(power_matvec_kernel, gmv, b256, 0, s, st, S, strideS, v, mv, n);
      hipLaunchKernelGGL(power_update_kernel, gb, b256, 0, s, st, v, mv, n, power_tol, max_power_iter);
    }
    hipLaunchKernelGGL(root_ridge_kernel, gc, b256, 0, s, st, S, strideS, n, ridge_eps);
    hipLaunchKernelGGL(root_zscale_kernel, gb, dim3(64), 0, s, st, p);
    if (planes && np == 2)
      hipLaunchKernelGGL(root_start_planes_kernel<2>, gc, b256, 0, s, st, S, strideS, pM[0], pT[0], pR[0], set_elems, n, n_pad,
                         p, kRootScaleM, scale_r);
    else if (planes)
      hipLaunchKernelGGL(root_start_planes_kernel<3>, gc, b256, 0, s, st, S, strideS, pM[0], pT[0], pR[0], set_elems, n, n_pad,
                         p, 1.f, 1.f);
    else
      hipLaunchKernelGGL(root_start_kernel, gc, b256, 0, s, st, S, strideS, Mb[0], Tb[0], out, strideOut, n, p);
    hipLaunchKernelGGL(root_begin_kernel, gb, dim3(64), 0, s, st, tol, max_iter);
  }
  if (!(phases & 2)) iters = 0;

  const int N = static_cast<int>(n);
  // The matrices of the iteration by number: two roots, two M, two T, four product buffers.  fp32 form: the first
  // root is the caller's `out`; plane form: all ten are plane sets of the workspace.
  enum { R0 = 0, R1, M0, M1, T0, T1, B0, B1, B2, B3, NBUF };
  float* fptr[NBUF] = {out, root1, Mb[0], Mb[1], Tb[0], Tb[1], buf[0], buf[1], buf[2], buf[3]};
  int64_t fstride[NBUF];
  for (int i = 0; i < NBUF; ++i) fstride[i] = nn;
  fstride[R0] = strideOut;
  __bf16* pptr[NBUF] = {pR[0], pR[1], pM[0], pM[1], pT[0], pT[1], pbuf[0], pbuf[1], pbuf[2], pbuf[3]};
  // C = A B for every matrix that still iterates.  next_T >= 0 (the product that forms M' only): the epilogue also
  // folds max |C - I| into the matrix's error word and writes the polynomial of the next step, (1 + 1/p) I - C / p.
  auto mm = [&](int ia, int ib, int ic, int next_T) {
    if (planes) {
      PlaneGemm g{};
      g.A = pptr[ia]; g.B = pptr[ib]; g.C = pptr[ic];
      g.sA = g.sB = g.sC = g.sC2 = set_elems;
      g.plane_elems = n_pad * n_pad;
      g.n = N; g.n_pad = static_cast<int>(n_pad); g.T = static_cast<int>(n_pad / kPlaneTile);
      g.active = st.active;
      g.overflow = st.ovf;
      if (next_T >= 0) {
        g.errword = st.errword;
        g.C2 = pptr[next_T];
        g.c2_scale = -1.0f / p; g.c2_diag = 1.0f + 1.0f / p;
      }
      // fp16 planes: the two roots carry scale_r, every other matrix kRootScaleM
      const float sa = ia <= R1 ? scale_r : kRootScaleM, sb = ib <= R1 ? scale_r : kRootScaleM;
      g.in_unscale = 1.0f / (sa * sb);
      g.c_scale = ic <= R1 ? scale_r : kRootScaleM;
      g.c2_plane_scale = kRootScaleM;
      return launch_plane_gemm(g, np, batch, s);
    }
    GemmParams g = make_gemm(0, 0, N, N, N, 1.f, fptr[ia], n, fptr[ib], n, 0.f, fptr[ic], n);
    g.sA = fstride[ia]; g.sB = fstride[ib]; g.sC = fstride[ic];
    g.active = st.active; g.active_stride = 1;
    g.split = g_root_split;
    // sums in chunks: the error of the root is set by the absolute rounding error of the first iterations' products
    // against the smallest eigenvalues of M (ridge_eps of the largest); a rank-deficient 1024 x 1024 statistic lost a
    // factor of six against LAPACK-grade fp32 products with one accumulator rounded at every matrix instruction
    g.chunked = 1;
    if (next_T >= 0) {
      g.absmax_out = st.errword; g.absmax_stride = 1; g.absmax_identity = 1;
      g.C2 = fptr[next_T]; g.ldc2 = n; g.sC2 = fstride[next_T];
      g.c2_scale = -1.0f / p; g.c2_diag = 1.0f + 1.0f / p;
    }
    // Every matrix of the iteration is a polynomial of the one symmetric statistic, so every product is symmetric up
    // to rounding: large ones compute the tiles on and below the diagonal only and mirror them (half the work; the
    // results are then exactly symmetric).  Small ones keep the full product.
    if (N >= kRootSymmetricMinDim) g.tile_mode = TILE_LOWER_MIRROR;
    return launch_gemm(g, batch, s);
  };
  auto copy = [&](int dst, int src) {
    const hipError_t e = planes
        ? hipMemcpyAsync(pptr[dst], pptr[src], sizeof(__bf16) * batch * set_elems, hipMemcpyDeviceToDevice, s)
        : hipMemcpyAsync(fptr[dst], fptr[src], sizeof(float) * batch * nn, hipMemcpyDeviceToDevice, s);
    return e == hipSuccess ? AK_OK : AK_ERR_LAUNCH;
  };
  // Iteration j of this call reads the buffer pair j % 2 (R, M, T) and writes the other one; an accepted step moves the
  // matrix's mark (st.par) there, so nothing is copied per step.  Every call starts with all marks on pair 0 and ends
  // by bringing the marked matrices back to it.
  for (int it = 0; it < iters; ++it) {
    const int a = it & 1, b = a ^ 1;
    const int T = T0 + a;
    int rc = mm(R0 + a, T, R0 + b, -1);                          // new_root = root T
    if (rc != AK_OK) return rc;
    // T^p with the multiplication order of MatPower
    int tp = -1;
    if ((p & (p - 1)) == 0) {
      int cur = T, which = B1;
      for (int done = 1; done < p; done *= 2) {
        rc = mm(cur, cur, which, -1);
        if (rc != AK_OK) return rc;
        cur = which;
        which = (which == B1) ? B2 : B1;
      }
      tp = cur;
    } else {
      int base = T, power = -1;     // squares ping-pong in B0 / B1, the running power in B2 / B3
      int sq = B0, pw = B2;
      for (int q = p; q > 0; q /= 2) {
        if (q & 1) {
          if (power < 0) {
            power = base;
          } else {
            rc = mm(base, power, pw, -1);
            if (rc != AK_OK) return rc;
            power = pw;
            pw = (pw == B2) ? B3 : B2;
          }
        }
        if (q / 2 > 0) {
          if (power == base && base != T) {      // a later square would overwrite the value `power` points at
            rc = copy(pw, base);
            if (rc != AK_OK) return rc;
            power = pw;
            pw = (pw == B2) ? B3 : B2;
          }
          rc = mm(base, base, sq, -1);
          if (rc != AK_OK) return rc;
          base = sq;
          sq = (sq == B0) ? B1 : B0;
        }
      }
      tp = power;
    }
    rc = mm(tp, M0 + a, M0 + b, T0 + b);                         // M' = T^p M, its error, the next T
    if (rc != AK_OK) return rc;
    hipLaunchKernelGGL(newton_decide_kernel, gb, dim3(64), 0, s, st, tol, max_iter, b);
  }
  if (iters > 0) {
    if (planes) {
      const int64_t words = set_elems / 2;
      hipLaunchKernelGGL(newton_gather_planes_kernel, gc, b256, 0, s, st, reinterpret_cast<uint32_t*>(pR[0]),
                         reinterpret_cast<const uint32_t*>(pR[1]), reinterpret_cast<uint32_t*>(pM[0]),
                         reinterpret_cast<const uint32_t*>(pM[1]), reinterpret_cast<uint32_t*>(pT[0]),
                         reinterpret_cast<const uint32_t*>(pT[1]), words);
    } else {
      hipLaunchKernelGGL(newton_gather_kernel, gc, b256, 0, s, st, out, strideOut, root1, Mb[0], Mb[1], Tb[0], Tb[1], n);
    }
    hipLaunchKernelGGL(newton_gathered_kernel, gb, dim3(64), 0, s, st);
  }
  // plane form: the caller's fp32 root is written with the statistics (the last part of a computation in parts)
  if ((phases & 4) && planes) {
    if (np == 2)
      hipLaunchKernelGGL(root_out_planes_kernel<2>, gc, b256, 0, s, pR[0], set_elems, out, strideOut, n, n_pad, st.zscale, p,
                         scale_r);
    else
      hipLaunchKernelGGL(root_out_planes_kernel<3>, gc, b256, 0, s, pR[0], set_elems, out, strideOut, n, n_pad, nullptr, p, 1.f);
  }
  if (phases & 4) hipLaunchKernelGGL(root_stats_kernel, gb, dim3(64), 0, s, st, stats);
  return check_launch();
}

}  // namespace ak

extern "C" int ak_inv_root_newton(float* S, int64_t n, int batch, int64_t strideS, int p, float ridge_eps,
                                  const float* v0, int max_power_iter, float power_tol, int max_iter, float tol,
                                  float* out, int64_t strideOut, float* stats, void* ws, size_t ws_bytes,
                                  ak_stream_t stream) {
  return ak::inv_root_run(7, max_iter, S, n, batch, strideS, p, ridge_eps, v0, max_power_iter, power_tol, max_iter, tol,
                          out, strideOut, stats, ws, ws_bytes, stream);
}

extern "C" int ak_inv_root_plane_format(int64_t n, int p, float ridge_eps) {
  if (n <= 0 || !ak::root_uses_planes(n)) return 0;
  return ak::root_fp16_scale(n, p, ridge_eps) > 0.f ? 2 : 3;
}

extern "C" size_t ak_inv_root_active_offset(int64_t n, int batch) {
  if (n <= 0 || batch <= 0) return 0;
  return ak::root_active_offset(n, batch);
}

extern "C" int ak_inv_root_newton_part(int phases, int iters, float* S, int64_t n, int batch, int64_t strideS, int p,
                                       float ridge_eps, const float* v0, int max_power_iter, float power_tol,
                                       int max_iter, float tol, float* out, int64_t strideOut, float* stats, void* ws,
                                       size_t ws_bytes, ak_stream_t stream) {
  if (phases < 1 || phases > 7 || iters < 0) return AK_ERR_ARG;
  return ak::inv_root_run(phases, iters, S, n, batch, strideS, p, ridge_eps, v0, max_power_iter, power_tol, max_iter,
                          tol, out, strideOut, stats, ws, ws_bytes, stream);
}

#ifdef AK_TUNING_HOOKS
namespace ak {
static __global__ void dbg_to_planes_kernel(const float* __restrict__ X, __bf16* __restrict__ P, int64_t n, int64_t n_pad) {
  const int64_t total = n_pad * n_pad;
  for (int64_t at = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; at < total; at += static_cast<int64_t>(gridDim.x) * 256) {
    const int64_t i = at / n_pad, j = at - i * n_pad;
    const float x = (i < n && j < n) ? X[i * n + j] : 0.f;
    unsigned short o[3];
    plane_bits<3>(x, o);
    unsigned short* Q = reinterpret_cast<unsigned short*>(P);
    const int64_t dst = plane_index(i, j, n_pad);
    Q[dst] = o[0]; Q[total + dst] = o[1]; Q[2 * total + dst] = o[2];
  }
}
}  // namespace ak

// Tuning builds only: C = A B for symmetric fp32 n x n matrices through the plane kernel (ws: 9 n_pad^2 bf16 + 1 float).
extern "C" int ak_debug_plane_product(const float* A, const float* B, float* C, int64_t n, void* ws, float* err) {
  using namespace ak;
  const int64_t n_pad = root_pad(n), set = 3 * n_pad * n_pad;
  __bf16* pa = static_cast<__bf16*>(ws);
  __bf16* pb = pa + set;
  __bf16* pc = pb + set;
  float* word = reinterpret_cast<float*>(pc + set);
  hipMemsetAsync(word, 0, 4, nullptr);
  hipLaunchKernelGGL(dbg_to_planes_kernel, dim3(512), dim3(256), 0, nullptr, A, pa, n, n_pad);
  hipLaunchKernelGGL(dbg_to_planes_kernel, dim3(512), dim3(256), 0, nullptr, B, pb, n, n_pad);
  PlaneGemm g{};
  g.A = pa; g.B = pb; g.C = pc;
  g.sA = g.sB = g.sC = g.sC2 = set;
  g.plane_elems = n_pad * n_pad;
  g.n = static_cast<int>(n); g.n_pad = static_cast<int>(n_pad); g.T = static_cast<int>(n_pad / kPlaneTile);
  g.errword = word;
  const int rc = launch_plane_gemm(g, 3, 1, nullptr);
  if (rc != AK_OK) return rc;
  hipLaunchKernelGGL(root_out_planes_kernel<3>, dim3(RCHUNKS, 1), dim3(256), 0, nullptr, pc, set, C, n * n, n, n_pad, nullptr, 1, 1.f);
  hipMemcpy(err, word, 4, hipMemcpyDeviceToHost);
  return check_launch();
}

// Tuning builds only: the smallest statistic that iterates on bf16 planes.
extern "C" void ak_debug_set_root_planes_min(int n) { ak::g_root_planes_min = n; }

// Tuning builds only: 0 = the fp32 MFMA kernel, 3 = the three-piece split kernel for the products of the Newton
// iteration.
extern "C" void ak_debug_set_root_split(int pieces) { ak::g_root_split = pieces; }
#endif
