// Kronecker preconditioning out <- scale * Binv G Ainv as back-to-back products in ONE launch, with the
// intermediate kept in the LDS (asdl/symmatrix.py:536-548 computes mat_B @ G @ mat_A with two torch.mm calls).
//
// Let the factor of the shorter side of G be Q (s x s, s <= 1024) and the other one P (L x L); both are symmetric.
// Seen with the long side as rows, G' = [L, s], the result is out' = P G' Q.  One work group owns R rows of out':
//   step 1   T[R, s]  = P[rows, :] G'          contraction over L, T stays in the LDS (R x s fp32, up to 128 KB)
//   step 2   out'[R, s] = scale * T Q          contraction over s, the T operand is read straight from the LDS
// so the [dB, dA] intermediate never exists in device memory.  R = 64 for s <= 512, else 32.  When the shorter side
// is the row side of G (dB < dA) the same kernel runs on the transposed view (G'[k][c] = G[c][k], P = Ainv,
// Q = Binv): element strides are parameters.
//
// True fp32 products (v_mfma_f32_32x32x2_f32): 4 waves, each owns 64 of the 256 columns of a chunk; operand tiles of
// 16 contraction steps are staged through the LDS with register prefetch.  P is read through its transpose
// (symmetric), which makes the loads of a k-row contiguous.  out must not alias G: every work group reads all of G.
#include "common.hpp"

namespace ak {

#define AK_LDSF __attribute__((address_space(3)))

constexpr int KF_BK = 16;           // contraction steps per staged tile
constexpr int KF_CW = 256;          // columns per chunk (4 waves x 2 MFMA tiles of 32)
constexpr int KF_GS = KF_CW + 1;    // row stride of the staged [16][256] tile (odd: both load mappings spread over the banks)

struct KronFusedParams {
  const float* P;      // [L, L], row stride L
  const float* Q;      // [s, s], row stride s
  const float* G;      // element (k, c) of the [L, s] view at G[k * gk + c * gc]
  float* out;          // same view, same strides
  int64_t gk, gc;
  int L, s;
  float scale;
};

template <int R>
struct KronFusedCfg {
  static constexpr int RT = R / 32;
  static constexpr int PT_FLOATS = KF_BK * R;             // staged P tile [16][R]
  static constexpr int GT_FLOATS = KF_BK * KF_GS;         // staged G' / Q tile [16][257]
  static size_t lds_bytes(int s) {
    const int sp = ((s + KF_CW - 1) / KF_CW) * KF_CW + 1;
    return (static_cast<size_t>(R) * sp + PT_FLOATS + GT_FLOATS) * sizeof(float);
  }
};

// GK1: the contraction index of G' is the contiguous one in memory (transposed view)
template <int R, bool GK1>
__global__ __launch_bounds__(256) void kron_precond_fused_kernel(KronFusedParams p) {
  using Cfg = KronFusedCfg<R>;
  constexpr int RT = Cfg::RT;
  extern __shared__ __attribute__((aligned(16))) float kf_smem[];
  const int s256 = ((p.s + KF_CW - 1) / KF_CW) * KF_CW, SP = s256 + 1;
  AK_LDSF float* Tp = (AK_LDSF float*)kf_smem;                  // [R][SP]
  AK_LDSF float* Pt = Tp + R * SP;                              // [16][R]
  AK_LDSF float* Gt = Pt + Cfg::PT_FLOATS;                      // [16][257]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, g = lane >> 5;
  const int r0 = blockIdx.x * R;

  // staging maps.  P tile: element (k, r) <- P[(k0 + k) * L + r0 + r], thread t holds r = t % R, k = t / R + j * (256 / R)
  constexpr int PK = 256 / R, PJ = KF_BK / PK;
  const int pr = tid % R, pk = tid / R;
  // G' tile: GK1 ? (k = t % 16, c = t / 16 + 16 j) : (c = t, k = j), 16 elements per thread either way
  float rp[PJ], rg[16];

  auto fetch_p = [&](int k0) {
#pragma unroll
    for (int j = 0; j < PJ; ++j) {
      const int k = k0 + pk + j * PK, r = r0 + pr;
      rp[j] = (k < p.L && r < p.L) ? p.P[static_cast<int64_t>(k) * p.L + r] : 0.f;
    }
  };
  auto stash_p = [&]() {
#pragma unroll
    for (int j = 0; j < PJ; ++j) Pt[(pk + j * PK) * R + pr] = rp[j];
  };
  // tile (k0.., c0..) of a [K, s] matrix with element strides (sk, sc); rows >= K and columns >= s read as zero
  auto fetch_g = [&](const float* __restrict__ M, int64_t sk, int64_t sc, int K, int k0, int c0, auto kfast_tag) {
    constexpr bool KFAST = decltype(kfast_tag)::value;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int k = k0 + (KFAST ? (tid & 15) : j), c = c0 + (KFAST ? (tid >> 4) + 16 * j : tid);
      rg[j] = (k < K && c < p.s) ? M[static_cast<int64_t>(k) * sk + static_cast<int64_t>(c) * sc] : 0.f;
    }
  };
  auto stash_g = [&](auto kfast_tag) {
    constexpr bool KFAST = decltype(kfast_tag)::value;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int k = KFAST ? (tid & 15) : j, c = KFAST ? (tid >> 4) + 16 * j : tid;
      Gt[k * KF_GS + c] = rg[j];
    }
  };

  floatx16 acc[RT][2];
  auto zero_acc = [&]() {
#pragma unroll
    for (int a = 0; a < RT; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  };

  // ---- step 1: T = P[rows, :] G'
  for (int c0 = 0; c0 < s256; c0 += KF_CW) {
    zero_acc();
    const int nk = (p.L + KF_BK - 1) / KF_BK;
    fetch_p(0);
    fetch_g(p.G, p.gk, p.gc, p.L, 0, c0, std::integral_constant<bool, GK1>{});
    for (int kt = 0; kt < nk; ++kt) {
      __syncthreads();                       // everybody is done with the previous tile
      stash_p();
      stash_g(std::integral_constant<bool, GK1>{});
      __syncthreads();
      if (kt + 1 < nk) {                     // the next tile's loads fly during this tile's products
        fetch_p((kt + 1) * KF_BK);
        fetch_g(p.G, p.gk, p.gc, p.L, (kt + 1) * KF_BK, c0, std::integral_constant<bool, GK1>{});
      }
#pragma unroll
      for (int kk = 0; kk < KF_BK; kk += 2) {
        float fa[RT], fb[2];
#pragma unroll
        for (int a = 0; a < RT; ++a) fa[a] = Pt[(kk + g) * R + 32 * a + l32];
#pragma unroll
        for (int b = 0; b < 2; ++b) fb[b] = Gt[(kk + g) * KF_GS + 64 * wave + 32 * b + l32];
#pragma unroll
        for (int a = 0; a < RT; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[a][b] = mfma_f32(fa[a], fb[b], acc[a][b]);
      }
    }
    // this chunk of T into the LDS panel (disjoint from the staged tiles)
#pragma unroll
    for (int a = 0; a < RT; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 32 * a + 8 * (r >> 2) + 4 * g + (r & 3), col = c0 + 64 * wave + 32 * b + l32;
          Tp[row * SP + col] = acc[a][b][r];
        }
  }

  // ---- step 2: out' = scale * T Q
  for (int c0 = 0; c0 < s256; c0 += KF_CW) {
    zero_acc();
    const int nk = (p.s + KF_BK - 1) / KF_BK;
    fetch_g(p.Q, p.s, 1, p.s, 0, c0, std::false_type{});
    for (int kt = 0; kt < nk; ++kt) {
      __syncthreads();                       // also orders the T panel writes of step 1 before its first read
      stash_g(std::false_type{});
      __syncthreads();
      if (kt + 1 < nk) fetch_g(p.Q, p.s, 1, p.s, (kt + 1) * KF_BK, c0, std::false_type{});
      const int k0 = kt * KF_BK;
#pragma unroll
      for (int kk = 0; kk < KF_BK; kk += 2) {
        float fa[RT], fb[2];
#pragma unroll
        for (int a = 0; a < RT; ++a) fa[a] = Tp[(32 * a + l32) * SP + k0 + kk + g];
#pragma unroll
        for (int b = 0; b < 2; ++b) fb[b] = Gt[(kk + g) * KF_GS + 64 * wave + 32 * b + l32];
#pragma unroll
        for (int a = 0; a < RT; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b) acc[a][b] = mfma_f32(fa[a], fb[b], acc[a][b]);
      }
    }
#pragma unroll
    for (int a = 0; a < RT; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int col = c0 + 64 * wave + 32 * b + l32;
        if (col >= p.s) continue;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = r0 + 32 * a + 8 * (r >> 2) + 4 * g + (r & 3);
          if (row < p.L) p.out[static_cast<int64_t>(row) * p.gk + static_cast<int64_t>(col) * p.gc] = p.scale * acc[a][b][r];
        }
      }
  }
}

constexpr int KRON_FUSED_MAX_SHORT = 1024;

template <int R, bool GK1>
static int kron_fused_launch(const KronFusedParams& p, hipStream_t stream) {
  auto kern = kron_precond_fused_kernel<R, GK1>;
  const size_t lds = KronFusedCfg<R>::lds_bytes(p.s);
  if (lds > 64 * 1024) {
    static size_t granted = 0;          // grows monotonically; a race sets it twice at worst
    if (granted < lds) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(160 * 1024)) != hipSuccess)
        return AK_ERR_LAUNCH;
      granted = 160 * 1024;
    }
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>((p.L + R - 1) / R)), dim3(256), lds, stream, p);
  return check_launch();
}

bool kron_fused_ok(int64_t dB, int64_t dA) { return (dB < dA ? dB : dA) <= KRON_FUSED_MAX_SHORT; }

// out <- scale * Binv G Ainv, G and out row-major [dB, dA], out != G.
int kron_precond_fused(const float* Binv, const float* Ainv, const float* G, float* out, int64_t dB, int64_t dA,
                       float scale, hipStream_t stream) {
  KronFusedParams p{};
  p.G = G; p.out = out; p.scale = scale;
  const bool rows_long = dB >= dA;           // long side = rows of G: P = Binv, Q = Ainv, natural view
  if (rows_long) { p.P = Binv; p.Q = Ainv; p.L = static_cast<int>(dB); p.s = static_cast<int>(dA); p.gk = dA; p.gc = 1; }
  else { p.P = Ainv; p.Q = Binv; p.L = static_cast<int>(dA); p.s = static_cast<int>(dB); p.gk = 1; p.gc = dA; }
  if (p.s <= 512) return rows_long ? kron_fused_launch<64, false>(p, stream) : kron_fused_launch<64, true>(p, stream);
  return rows_long ? kron_fused_launch<32, false>(p, stream) : kron_fused_launch<32, true>(p, stream);
}

}  // namespace ak

extern "C" int64_t ak_kron_precond_fused_max_short(void) { return ak::KRON_FUSED_MAX_SHORT; }
