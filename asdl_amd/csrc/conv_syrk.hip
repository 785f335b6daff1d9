// A <- beta*A + alpha * sum over output positions of patch patch^T, with the im2col unfold
// fused: the patch matrix [n, c*kh*kw, h_out*w_out] never exists in memory.
//
// Row index of A: i = (c, ky, kx).  Contraction index: k = (n, oy, ox).  Consecutive ox are
// consecutive in NCHW memory, so the contraction index is the contiguous one and an MFMA
// operand (8 consecutive k for one i) is 16 contiguous bytes -- provided it is 16-byte
// aligned in LDS.  The kernel therefore stages, per panel of 64*TI rows of A and per block of
// R x WC output positions, one LDS row for every (channel, kx, input row):
//     plane[c][kx][r][q] = x[n, c, oy0*sh - ph + r, (ox0 + q)*sw + kx - pw]   (0 outside)
// i.e. the kx shift (and the sw decimation) is applied on the way in, with unaligned 16-byte
// global loads, and every MFMA fragment afterwards is one aligned ds_read_b128 at
//     base(i) + (oy_local*sh)*RS + 8*u,   base(i) = ((c_local*kw + kx)*RI + ky)*RS.
// The ky shift is a whole-row offset and costs nothing.  The k-space is padded to a multiple
// of 8 per output row with zeros.  kh = kw = 1 with H = 1 is the plain "X X^T, contraction
// contiguous" case used for Conv2d.cov_kron_B and for Shampoo's G G^T.
#include "common.hpp"

namespace ak {

struct ConvSyrkParams {
  const void* x;
  int64_t N, C, H, W;
  int kh, kw, sh, sw, ph, pw, Ho, Wo;
  int64_t d;
  float alpha, beta;
  float* A;
  int64_t lda;
  float* ws;
  int T, nsplit;
  int KK;        // kh*kw
  int R;         // output rows per stage
  int WC;        // output columns per stage (multiple of 8)
  int U;         // WC / 8 k-units per output row
  int RI;        // input rows per stage = (R-1)*sh + kh
  int RS;        // LDS row stride in elements
  int NCmax;     // channels a panel can touch
  int panel_elems;
  int RB, CB;    // row blocks per image, column chunks per row
  int64_t total_stages, stages_per_split;
  uint32_t mU, mKK, mKw, mRI, mKwRI, mCPR, mCB, mRBCB;   // magic multipliers for division
  int RP, dcl, dkx, dr;   // LDS rows staged per pass of the work group, and that step decomposed as (channel, kx, row)
};

__host__ __device__ inline uint32_t make_magic(uint32_t d) { return static_cast<uint32_t>((0x100000000ull + d - 1) / d); }
// exact for x * d < 2^32
__device__ __forceinline__ uint32_t fastdiv(uint32_t x, uint32_t magic, uint32_t d) {
  return d == 1 ? x : __umulhi(x, magic);
}

typedef uint4 __attribute__((aligned(2))) uint4_a2;
typedef uint4 __attribute__((aligned(4))) uint4_a4;

template <typename T> struct Elem;
template <> struct Elem<uint16_t> { static constexpr int E = 8; typedef uint4_a2 vec_u; };
template <> struct Elem<float> { static constexpr int E = 4; typedef uint4_a4 vec_u; };

// Fills one panel's planes for the stage (n, oy0, ox0).  Thread t owns 16-byte chunk t % CPR of LDS rows
// t / CPR, t / CPR + RP, ...; the row index is decoded to (channel, kx, input row) once and then advanced
// with carries, so the loop body has no divisions.
template <typename T>
__device__ __forceinline__ void stage_panel(T* __restrict__ plane, const ConvSyrkParams& p, const T* __restrict__ x,
                                            int64_t n, int c_lo, int nc, int oy0, int ox0, int R_eff, int W_eff,
                                            int tid) {
  constexpr int E = Elem<T>::E;
  const int CPR = p.WC / E;
  const int row0 = static_cast<int>(fastdiv(tid, p.mCPR, CPR));
  if (row0 >= p.RP) return;
  const int m = tid - row0 * CPR;
  const int kwRI = p.kw * p.RI;
  const int total_rows = nc * kwRI;
  int cl = static_cast<int>(fastdiv(row0, p.mKwRI, kwRI));
  const int t2 = row0 - cl * kwRI;
  int kx = static_cast<int>(fastdiv(t2, p.mRI, p.RI));
  int r = t2 - kx * p.RI;
  const int RI_eff = (R_eff - 1) * p.sh + p.kh;
  const int q0 = m * E;
  const int xq = (ox0 + q0) * p.sw - p.pw;
  const int iy0 = oy0 * p.sh - p.ph;
  const bool q_in = q0 < W_eff, q_full = q0 + E <= W_eff;
  const T* __restrict__ img = x + n * p.C * p.H * p.W;
  T* __restrict__ dst = plane + row0 * p.RS + q0;
  const int dst_step = p.RP * p.RS;
  for (int rs = row0; rs < total_rows; rs += p.RP, dst += dst_step) {
    const int iy = iy0 + r;
    const int x0 = xq + kx;
    uint4 v = {0u, 0u, 0u, 0u};
    if (q_in && r < RI_eff && iy >= 0 && iy < p.H) {
      const T* src = img + (static_cast<int64_t>(c_lo + cl) * p.H + iy) * p.W;
      const bool inner = q_full && (x0 >= 0);
      if (p.sw == 1 && inner && x0 + E <= p.W) {
        v = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0);
      } else if (p.sw == 2 && inner && x0 + 2 * E <= p.W) {
        const uint4 lo = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0);
        const uint4 hi = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0 + E);
        if constexpr (sizeof(T) == 2) {
          v.x = (lo.x & 0xffffu) | (lo.y << 16);
          v.y = (lo.z & 0xffffu) | (lo.w << 16);
          v.z = (hi.x & 0xffffu) | (hi.y << 16);
          v.w = (hi.z & 0xffffu) | (hi.w << 16);
        } else {
          v.x = lo.x; v.y = lo.z; v.z = hi.x; v.w = hi.z;
        }
      } else {
        alignas(16) T tmp[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const int xe = x0 + e * p.sw;
          tmp[e] = (q0 + e < W_eff && xe >= 0 && xe < p.W) ? src[xe] : T(0);
        }
        v = *reinterpret_cast<uint4*>(tmp);
      }
    }
    *reinterpret_cast<uint4*>(dst) = v;
    r += p.dr; kx += p.dkx; cl += p.dcl;
    if (r >= p.RI) { r -= p.RI; kx += 1; }
    if (kx >= p.kw) { kx -= p.kw; cl += 1; }
  }
}

template <typename T, int TI>
__global__ __launch_bounds__(256) void conv_syrk_kernel(ConvSyrkParams p) {
  constexpr int BT = 64 * TI;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* planeI = reinterpret_cast<T*>(smem);
  T* planeJ = planeI + p.panel_elems;
  T* zero_unit = planeJ + p.panel_elems;   // 8 elements of zeros

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int g = lane >> 5, l32 = lane & 31;
  int ti, tj;
  decode_upper_tile(blockIdx.x, p.T, ti, tj);
  const bool diag = (ti == tj);
  const int64_t i0 = static_cast<int64_t>(ti) * BT, j0 = static_cast<int64_t>(tj) * BT;
  const T* __restrict__ x = static_cast<const T*>(p.x);

  auto chan_range = [&](int64_t r0, int& c_lo, int& nc) {
    int64_t last = r0 + BT - 1;
    if (last > p.d - 1) last = p.d - 1;
    c_lo = static_cast<int>(fastdiv(static_cast<uint32_t>(r0), p.mKK, p.KK));
    nc = static_cast<int>(fastdiv(static_cast<uint32_t>(last), p.mKK, p.KK)) - c_lo + 1;
  };
  int cI, ncI, cJ, ncJ;
  chan_range(i0, cI, ncI);
  chan_range(j0, cJ, ncJ);
  if (diag) planeJ = planeI;

  auto frag_base = [&](int64_t row, int c_lo) {
    if (row > p.d - 1) row = p.d - 1;
    const uint32_t i = static_cast<uint32_t>(row);
    const uint32_t c = fastdiv(i, p.mKK, p.KK);
    const uint32_t rem = i - c * p.KK;
    const uint32_t ky = fastdiv(rem, p.mKw, p.kw);
    const uint32_t kx = rem - ky * p.kw;
    return static_cast<int>((((c - c_lo) * p.kw + kx) * p.RI + ky) * p.RS);
  };
  int baseI[TI], baseJ[TI];
#pragma unroll
  for (int a = 0; a < TI; ++a) baseI[a] = frag_base(i0 + 32 * TI * wr + 32 * a + l32, cI);
#pragma unroll
  for (int b = 0; b < TI; ++b) baseJ[b] = frag_base(j0 + 32 * TI * wc + 32 * b + l32, cJ);

  if (tid < 8) zero_unit[tid] = T(0);

  floatx16 acc[TI][TI];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TI; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const int64_t s_begin = static_cast<int64_t>(blockIdx.y) * p.stages_per_split;
  int64_t s_end = s_begin + p.stages_per_split;
  if (s_end > p.total_stages) s_end = p.total_stages;
  const int RBCB = p.RB * p.CB;

  for (int64_t s = s_begin; s < s_end; ++s) {
    const uint32_t s32 = static_cast<uint32_t>(s);
    const uint32_t n = fastdiv(s32, p.mRBCB, RBCB);
    const uint32_t t2 = s32 - n * RBCB;
    const uint32_t rb = fastdiv(t2, p.mCB, p.CB);
    const uint32_t cb = t2 - rb * p.CB;
    const int oy0 = rb * p.R, ox0 = cb * p.WC;
    const int R_eff = min(p.R, p.Ho - oy0);
    const int W_eff = min(p.WC, p.Wo - ox0);

    __syncthreads();
    stage_panel<T>(planeI, p, x, n, cI, ncI, oy0, ox0, R_eff, W_eff, tid);
    if (!diag) stage_panel<T>(planeJ, p, x, n, cJ, ncJ, oy0, ox0, R_eff, W_eff, tid);
    __syncthreads();

    const int nunits = R_eff * p.U;
    for (int f0 = 0; f0 < nunits; f0 += 2) {
      const int f = f0 + g;
      const bool valid = f < nunits;
      const uint32_t r = fastdiv(static_cast<uint32_t>(f), p.mU, p.U);
      const int off = r * p.sh * p.RS + (f - r * p.U) * 8;
      if constexpr (sizeof(T) == 2) {
        bf16x8 fa[TI], fb[TI];
#pragma unroll
        for (int a = 0; a < TI; ++a)
          fa[a] = *reinterpret_cast<const bf16x8*>(valid ? planeI + baseI[a] + off : zero_unit);
#pragma unroll
        for (int b = 0; b < TI; ++b)
          fb[b] = *reinterpret_cast<const bf16x8*>(valid ? planeJ + baseJ[b] + off : zero_unit);
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
          for (int b = 0; b < TI; ++b) acc[a][b] = mfma_bf16(fa[a], fb[b], acc[a][b]);
      } else {
        floatx4 fa[TI][2], fb[TI][2];
#pragma unroll
        for (int a = 0; a < TI; ++a) {
          const floatx4* q = reinterpret_cast<const floatx4*>(valid ? planeI + baseI[a] + off : zero_unit);
          fa[a][0] = q[0];
          fa[a][1] = q[1];
        }
#pragma unroll
        for (int b = 0; b < TI; ++b) {
          const floatx4* q = reinterpret_cast<const floatx4*>(valid ? planeJ + baseJ[b] + off : zero_unit);
          fb[b][0] = q[0];
          fb[b][1] = q[1];
        }
#pragma unroll
        for (int m = 0; m < 8; ++m)
#pragma unroll
          for (int a = 0; a < TI; ++a)
#pragma unroll
            for (int b = 0; b < TI; ++b)
              acc[a][b] = mfma_f32(fa[a][m >> 2][m & 3], fb[b][m >> 2][m & 3], acc[a][b]);
      }
    }
  }

  if (p.nsplit == 1) {
    syrk_epilogue<TI, TI>(acc, p.A, p.lda, p.d, i0 + 32 * TI * wr, j0 + 32 * TI * wc, diag, p.alpha, p.beta, lane);
  } else {
    store_partial<TI, TI>(acc, p.ws + (static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (BT * BT), tid);
  }
}

// Host-side geometry shared by the launch and the workspace query.
struct ConvPlan {
  ConvSyrkParams p;
  int BT;
  size_t lds_bytes;
  int64_t ntiles;
  size_t ws_need;
};

static int tile_rows_for(int64_t d) { return d <= 64 ? 64 : 128; }

static bool make_plan(ConvPlan& plan, int esize, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                      int sw, int ph, int pw) {
  ConvSyrkParams& p = plan.p;
  const int BT = tile_rows_for(C * kh * kw);
  plan.BT = BT;
  bool flat = false;
  if (kh == 1 && kw == 1 && ph == 0 && pw == 0 && sh == 1 && sw == 1) {  // positions are contiguous: flatten
    W = H * W;
    H = 1;
    flat = true;
  }
  const int64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
  if (Ho <= 0 || Wo <= 0) return false;
  p.N = N; p.C = C; p.H = H; p.W = W;
  p.kh = kh; p.kw = kw; p.sh = sh; p.sw = sw; p.ph = ph; p.pw = pw;
  p.Ho = static_cast<int>(Ho); p.Wo = static_cast<int>(Wo);
  p.KK = kh * kw;
  p.d = C * p.KK;
  const int wc_max = (flat && esize == 2) ? 128 : 64;
  int WC = static_cast<int>(((Wo + 7) / 8) * 8);
  if (WC > wc_max) WC = wc_max;
  p.WC = WC;
  p.U = WC / 8;
  int pad = 8;
  if (((WC + pad) * esize / 16) % 2 == 0) pad += 16 / esize;   // odd number of 16-byte units per LDS row
  p.RS = WC + pad;
  int ncmax = (BT - 1 + p.KK - 1) / p.KK + 1;
  if (ncmax > C) ncmax = static_cast<int>(C);
  p.NCmax = ncmax;
  const size_t budget = 80 * 1024 - 64;     // two work groups per CU
  int R = 1;
  for (int cand = 1; cand <= Ho && cand * WC <= 1024; ++cand) {
    const int RI = (cand - 1) * sh + kh;
    const size_t bytes = 2ull * ncmax * kw * RI * p.RS * esize;
    if (bytes <= budget) R = cand; else break;
  }
  {  // equal-sized row blocks: no short last block
    const int64_t nrb = (Ho + R - 1) / R;
    R = static_cast<int>((Ho + nrb - 1) / nrb);
  }
  p.R = R;
  p.RI = (R - 1) * sh + kh;
  p.panel_elems = ncmax * kw * p.RI * p.RS;
  plan.lds_bytes = 2ull * p.panel_elems * esize + 64;
  if (plan.lds_bytes > 160 * 1024) return false;
  p.RB = static_cast<int>((Ho + R - 1) / R);
  p.CB = static_cast<int>((Wo + WC - 1) / WC);
  p.total_stages = N * p.RB * p.CB;
  if (p.total_stages >= (1ll << 31) || p.d >= (1ll << 24)) return false;
  if (p.total_stages * p.RB * p.CB >= (1ll << 32)) return false;   // exactness of the magic division
  const int64_t Tn = (p.d + BT - 1) / BT;
  p.T = static_cast<int>(Tn);
  plan.ntiles = Tn * (Tn + 1) / 2;
  const int64_t ksteps_per_stage = (static_cast<int64_t>(R) * WC + 31) / 32;
  int nsplit = pick_nsplit(plan.ntiles, p.total_stages * ksteps_per_stage);
  if (nsplit > p.total_stages) nsplit = static_cast<int>(p.total_stages);
  if (nsplit < 1) nsplit = 1;
  p.stages_per_split = (p.total_stages + nsplit - 1) / nsplit;
  if (p.stages_per_split < 1) p.stages_per_split = 1;
  nsplit = static_cast<int>((p.total_stages + p.stages_per_split - 1) / p.stages_per_split);
  if (nsplit < 1) nsplit = 1;
  p.nsplit = nsplit;
  plan.ws_need = nsplit > 1 ? static_cast<size_t>(nsplit) * plan.ntiles * BT * BT * sizeof(float) : 0;
  const int CPR = WC / (16 / esize);
  p.RP = 256 / CPR;
  {
    const int kwRI = kw * p.RI;
    p.dcl = p.RP / kwRI;
    const int rem = p.RP - p.dcl * kwRI;
    p.dkx = rem / p.RI;
    p.dr = rem - p.dkx * p.RI;
  }
  p.mU = make_magic(p.U); p.mKK = make_magic(p.KK); p.mKw = make_magic(kw); p.mRI = make_magic(p.RI);
  p.mKwRI = make_magic(kw * p.RI); p.mCPR = make_magic(CPR); p.mCB = make_magic(p.CB);
  p.mRBCB = make_magic(p.RB * p.CB);
  return true;
}

template <typename T, int TI>
static int launch_conv_syrk_t(ConvPlan& plan, hipStream_t stream) {
  auto kern = conv_syrk_kernel<T, TI>;
  if (plan.lds_bytes > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(plan.lds_bytes)) != hipSuccess)
      return AK_ERR_LAUNCH;
  }
  dim3 grid(static_cast<unsigned>(plan.ntiles), static_cast<unsigned>(plan.p.nsplit));
  hipLaunchKernelGGL(kern, grid, dim3(256), plan.lds_bytes, stream, plan.p);
  if (plan.p.nsplit > 1)
    hipLaunchKernelGGL((syrk_finalize_kernel<TI, TI>), dim3(static_cast<unsigned>(plan.ntiles), 4 * TI * TI), dim3(256), 0, stream,
                       static_cast<const float*>(plan.p.ws), plan.p.nsplit, plan.p.T, plan.p.A, plan.p.lda, plan.p.d,
                       plan.p.alpha, plan.p.beta);
  return check_launch();
}

template <typename T>
static int launch_conv_syrk(ConvPlan& plan, hipStream_t stream) {
  return plan.BT == 64 ? launch_conv_syrk_t<T, 1>(plan, stream) : launch_conv_syrk_t<T, 2>(plan, stream);
}

}  // namespace ak

extern "C" size_t ak_conv_syrk_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw,
                                        int ph, int pw) {
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 || ph < 0 || pw < 0) return 0;
  ak::ConvPlan a, b;
  size_t need = 0;
  if (ak::make_plan(a, 2, N, C, H, W, kh, kw, sh, sw, ph, pw)) need = a.ws_need;
  if (ak::make_plan(b, 4, N, C, H, W, kh, kw, sh, sw, ph, pw) && b.ws_need > need) need = b.ws_need;
  return need;
}

extern "C" int ak_conv_syrk(const void* x, int dtype, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                            int sw, int ph, int pw, float alpha, float beta, float* A, int64_t lda, void* ws,
                            size_t ws_bytes, ak_stream_t stream) {
  if (x == nullptr || A == nullptr || N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 ||
      sw <= 0 || ph < 0 || pw < 0)
    return AK_ERR_ARG;
  if (dtype != AK_BF16 && dtype != AK_F32) return AK_ERR_ARG;
  ak::ConvPlan plan;
  if (!ak::make_plan(plan, dtype == AK_BF16 ? 2 : 4, N, C, H, W, kh, kw, sh, sw, ph, pw)) return AK_ERR_UNSUPPORTED;
  if (lda < plan.p.d) return AK_ERR_ARG;
  if (plan.ws_need > 0 && (ws == nullptr || ws_bytes < plan.ws_need)) return AK_ERR_WORKSPACE;
  plan.p.x = x; plan.p.alpha = alpha; plan.p.beta = beta; plan.p.A = A; plan.p.lda = lda;
  plan.p.ws = static_cast<float*>(ws);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == AK_BF16 ? ak::launch_conv_syrk<uint16_t>(plan, s) : ak::launch_conv_syrk<float>(plan, s);
}
