// C <- beta*C + alpha * X^T X for a row-major X[M, d] (the contraction index is the strided one).
//
// One work group (4 waves, 2x2) owns one BT x BT tile of the upper triangle of C and, with
// split-K, one slice of the M rows.  Panels of X are copied global -> LDS as they lie in
// memory ([k][i], i contiguous, 16-byte vectors).
//   bf16: MFMA 32x32x16 needs 8 consecutive k per lane; ds_read_b64_tr_b16 transposes on the
//         way out of LDS, so no transposed copy of X is ever made.
//   fp32: MFMA 32x32x2 takes one k per lane; plain ds_read_b32 along i is conflict free.
// Both operands of the rank-k update come from the same matrix, so diagonal tiles load a
// single panel.
#include "common.hpp"

namespace ak {

template <typename T> struct TnCfg;
template <> struct TnCfg<uint16_t> { static constexpr int BK = 32, PAD = 16, E = 8; };
template <> struct TnCfg<float> { static constexpr int BK = 16, PAD = 4, E = 4; };

struct SyrkTnParams {
  const void* X;
  int64_t M, d, ldx;
  float alpha, beta;
  float* C;
  int64_t ldc;
  float* ws;
  int T, nsplit;
  int64_t rows_per_split;
};

template <typename T>
__device__ __forceinline__ uint4 load_chunk(const T* __restrict__ X, int64_t row, int64_t col, int64_t row_end,
                                            int64_t d, int64_t ldx, bool vec_ok) {
  constexpr int E = TnCfg<T>::E;
  uint4 v = {0u, 0u, 0u, 0u};
  if (row < row_end && col < d) {
    const T* src = X + row * ldx + col;
    if (vec_ok && col + E <= d) {
      v = *reinterpret_cast<const uint4*>(src);
    } else {
      alignas(16) T tmp[E];
#pragma unroll
      for (int e = 0; e < E; ++e) tmp[e] = (col + e < d) ? src[e] : T(0);
      v = *reinterpret_cast<uint4*>(tmp);
    }
  }
  return v;
}

template <typename T, int TI>
__global__ __launch_bounds__(256, 2) void syrk_tn_kernel(SyrkTnParams p) {
  constexpr int BT = 64 * TI;
  constexpr int BK = TnCfg<T>::BK, PAD = TnCfg<T>::PAD, E = TnCfg<T>::E;
  constexpr int LDSS = BT + PAD;                 // elements per k-row in LDS
  constexpr int CPR = BT / E;                    // 16-byte chunks per k-row
  constexpr int CHUNKS = BK * CPR / 256;         // chunks per thread per panel
  constexpr int PANEL = BK * LDSS;               // elements per panel buffer
  static_assert(BK * CPR % 256 == 0, "panel must split evenly");
  extern __shared__ __attribute__((aligned(16))) unsigned char tn_smem[];
  T* lds = reinterpret_cast<T*>(tn_smem);        // [buffer][panel][BK * LDSS]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  int ti, tj;
  decode_upper_tile(blockIdx.x, p.T, ti, tj);
  const bool diag = (ti == tj);
  const int64_t i0 = static_cast<int64_t>(ti) * BT, j0 = static_cast<int64_t>(tj) * BT;
  const int64_t k_begin = static_cast<int64_t>(blockIdx.y) * p.rows_per_split;
  int64_t k_end = k_begin + p.rows_per_split;
  if (k_end > p.M) k_end = p.M;
  const int nk = k_begin < k_end ? static_cast<int>((k_end - k_begin + BK - 1) / BK) : 0;

  const T* __restrict__ X = static_cast<const T*>(p.X);
  const bool vec_ok = (p.ldx % E == 0) && ((reinterpret_cast<uintptr_t>(X) & 15) == 0);
  // whole panels inside the matrix and aligned: plain vector loads, no per-chunk tests
  const bool fast = vec_ok && (j0 + BT <= p.d);   // j0 >= i0, so this covers the I panel too

  floatx16 acc[TI][TI];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TI; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  uint4 regI[CHUNKS], regJ[CHUNKS];
  auto fetch = [&](int kt) {
    const int64_t kb = k_begin + static_cast<int64_t>(kt) * BK;
    if (fast && kb + BK <= k_end) {
#pragma unroll
      for (int u = 0; u < CHUNKS; ++u) {
        const int c = tid + 256 * u;
        const T* src = X + (kb + c / CPR) * p.ldx + (c % CPR) * E;
        regI[u] = *reinterpret_cast<const uint4*>(src + i0);
        if (!diag) regJ[u] = *reinterpret_cast<const uint4*>(src + j0);
      }
    } else {
#pragma unroll
      for (int u = 0; u < CHUNKS; ++u) {
        const int c = tid + 256 * u;
        const int row = c / CPR, cc = c % CPR;
        regI[u] = load_chunk<T>(X, kb + row, i0 + cc * E, k_end, p.d, p.ldx, vec_ok);
        if (!diag) regJ[u] = load_chunk<T>(X, kb + row, j0 + cc * E, k_end, p.d, p.ldx, vec_ok);
      }
    }
  };
  auto stash = [&](int buf) {
    T* pI = lds + (2 * buf) * PANEL;
    T* pJ = pI + PANEL;
#pragma unroll
    for (int u = 0; u < CHUNKS; ++u) {
      const int c = tid + 256 * u;
      const int row = c / CPR, cc = c % CPR;
      *reinterpret_cast<uint4*>(&pI[row * LDSS + cc * E]) = regI[u];
      if (!diag) *reinterpret_cast<uint4*>(&pJ[row * LDSS + cc * E]) = regJ[u];
    }
  };

  if (nk > 0) {
    fetch(0);
    stash(0);
  }
  __syncthreads();

  const int g = lane >> 5, l32 = lane & 31;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) fetch(kt + 1);
    const T* pI = lds + (2 * buf) * PANEL;
    const T* pJ = diag ? pI : pI + PANEL;
    if constexpr (sizeof(T) == 2) {
      const int half = (lane >> 4) & 1, j16 = lane & 15;
      const int frag_off = (8 * g + (j16 >> 2)) * LDSS + 16 * half + 4 * (j16 & 3);
      const T* qI = pI + frag_off + 32 * TI * wr;
      const T* qJ = pJ + frag_off + 32 * TI * wc;
      auto read = [&](bf16x8 (&fa)[TI], bf16x8 (&fb)[TI], int kk) {
#pragma unroll
        for (int a = 0; a < TI; ++a) {
          const T* q = qI + kk * LDSS + 32 * a;
          fa[a] = pack_bf16x8(lds_read_tr16(q), lds_read_tr16(q + 4 * LDSS));
        }
#pragma unroll
        for (int b = 0; b < TI; ++b) {
          const T* q = qJ + kk * LDSS + 32 * b;
          fb[b] = pack_bf16x8(lds_read_tr16(q), lds_read_tr16(q + 4 * LDSS));
        }
      };
      auto mma = [&](const bf16x8 (&fa)[TI], const bf16x8 (&fb)[TI]) {
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
          for (int b = 0; b < TI; ++b) acc[a][b] = mfma_bf16(fa[a], fb[b], acc[a][b]);
      };
      // ping-pong fragment registers: the reads of one k-step fly during the MFMAs of the previous one
      bf16x8 fa0[TI], fb0[TI], fa1[TI], fb1[TI];
      read(fa0, fb0, 0);
#pragma unroll
      for (int kk = 0; kk < BK; kk += 32) {
        read(fa1, fb1, kk + 16);
        mma(fa0, fb0);
        if (kk + 32 < BK) read(fa0, fb0, kk + 32);
        mma(fa1, fb1);
      }
    } else {
#pragma unroll
      for (int m = 0; m < BK / 2; ++m) {
        const int k = 2 * m + g;
        float fa[TI], fb[TI];
#pragma unroll
        for (int a = 0; a < TI; ++a) fa[a] = pI[k * LDSS + 32 * TI * wr + 32 * a + l32];
#pragma unroll
        for (int b = 0; b < TI; ++b) fb[b] = pJ[k * LDSS + 32 * TI * wc + 32 * b + l32];
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
          for (int b = 0; b < TI; ++b) acc[a][b] = mfma_f32(fa[a], fb[b], acc[a][b]);
      }
    }
    if (kt + 1 < nk) stash(buf ^ 1);
    __syncthreads();
  }

  if (p.nsplit == 1) {
    syrk_epilogue<TI, TI>(acc, p.C, p.ldc, p.d, i0 + 32 * TI * wr, j0 + 32 * TI * wc, diag, p.alpha, p.beta, lane);
  } else {
    store_partial<TI, TI>(acc, p.ws + (static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (BT * BT), tid);
  }
}

template <typename T>
static int launch_syrk_tn(const void* X, int64_t M, int64_t d, int64_t ldx, float alpha, float beta, float* C,
                          int64_t ldc, void* ws, size_t ws_bytes, hipStream_t stream) {
  constexpr int TI = 2, BT = 64 * TI, BK = TnCfg<T>::BK;
  const int64_t Tn = (d + BT - 1) / BT;
  const int64_t ntiles = Tn * (Tn + 1) / 2;
  const int64_t ksteps = (M + BK - 1) / BK;
  int nsplit = pick_nsplit(ntiles, ksteps);
  int64_t steps_per_split = (ksteps + nsplit - 1) / nsplit;
  if (steps_per_split < 1) steps_per_split = 1;
  nsplit = static_cast<int>((ksteps + steps_per_split - 1) / steps_per_split);
  if (nsplit < 1) nsplit = 1;
  if (nsplit > 1) {
    const size_t need = static_cast<size_t>(nsplit) * ntiles * BT * BT * sizeof(float);
    if (ws == nullptr || ws_bytes < need) return AK_ERR_WORKSPACE;
  }
  SyrkTnParams p;
  p.X = X; p.M = M; p.d = d; p.ldx = ldx; p.alpha = alpha; p.beta = beta; p.C = C; p.ldc = ldc;
  p.ws = static_cast<float*>(ws); p.T = static_cast<int>(Tn); p.nsplit = nsplit;
  p.rows_per_split = steps_per_split * BK;
  dim3 grid(static_cast<unsigned>(ntiles), static_cast<unsigned>(nsplit));
  constexpr size_t lds_bytes = 4ull * BK * (BT + TnCfg<T>::PAD) * sizeof(T);
  auto kern = syrk_tn_kernel<T, TI>;
  if (lds_bytes > 64 * 1024) {
    static bool attr_set = false;     // idempotent; a benign race sets it twice at worst
    if (!attr_set) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              static_cast<int>(lds_bytes)) != hipSuccess)
        return AK_ERR_LAUNCH;
      attr_set = true;
    }
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), lds_bytes, stream, p);
  if (nsplit > 1)
    hipLaunchKernelGGL((syrk_finalize_kernel<TI, TI>), dim3(static_cast<unsigned>(ntiles), 4 * TI * TI), dim3(256), 0, stream,
                       static_cast<const float*>(ws), nsplit, static_cast<int>(Tn), C, ldc, d, alpha, beta);
  return check_launch();
}

}  // namespace ak

extern "C" size_t ak_syrk_tn_ws_bytes(int64_t M, int64_t d) {
  if (M <= 0 || d <= 0) return 0;
  const int64_t Tn = (d + 127) / 128;
  const int64_t ntiles = Tn * (Tn + 1) / 2;
  // upper bound over both dtypes (bf16 has the fewer k-steps, fp32 the more)
  const int ns = ak::pick_nsplit(ntiles, (M + 15) / 16);
  const size_t staged = ns > 1 ? static_cast<size_t>(ns) * ntiles * 128 * 128 * sizeof(float) : 0;
  const size_t direct = d % 8 == 0 ? ak::syrk_dtl_plain_ws_bytes(M, d, d) : 0;
  return staged > direct ? staged : direct;
}

extern "C" int ak_syrk_tn(const void* X, int dtype, int64_t M, int64_t d, int64_t ldx, float alpha, float beta,
                          float* C, int64_t ldc, void* ws, size_t ws_bytes, ak_stream_t stream) {
  if (X == nullptr || C == nullptr || M < 0 || d <= 0 || ldx < d || ldc < d) return AK_ERR_ARG;
  if (!ak::syrk_beta_ok(beta, d, ldc)) return AK_ERR_UNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == AK_BF16 && ak::syrk_dtl_plain_ok(X, M, d, ldx)) {
    const int rc = ak::syrk_dtl_plain(X, M, d, ldx, alpha, beta, C, ldc, ws, ws_bytes, s);
    if (rc != AK_ERR_UNSUPPORTED && rc != AK_ERR_WORKSPACE) return rc;
  }
  if (dtype == AK_BF16) return ak::launch_syrk_tn<uint16_t>(X, M, d, ldx, alpha, beta, C, ldc, ws, ws_bytes, s);
  if (dtype == AK_F32) return ak::launch_syrk_tn<float>(X, M, d, ldx, alpha, beta, C, ldc, ws, ws_bytes, s);
  return AK_ERR_ARG;
}
