// fp32 MFMA GEMM tile kernel shared by the dense products (precondition, Newton iteration)
// and by the blocked Cholesky inverse, which needs triangular-aware contraction ranges.
//
// C[M,N] <- alpha * op(A) op(B) + beta * C, row-major, v_mfma_f32_32x32x2_f32 (true fp32 products,
// fp32 accumulation).  One work group = 4 waves (2x2) = one 128x128 tile, BK = 16.
// An operand whose contraction index is contiguous in memory is kept in LDS as [row][16 + 4] and
// read as two ds_read_b128 per lane (8 k values); one whose row/column index is contiguous is kept
// as [k][128 + 4] and read with conflict-free ds_read_b32.  No transposed copies are made.
#pragma once
#include "common.hpp"

namespace ak {

enum KMode {
  K_FULL = 0,
  K_LE_J = 1,     // contraction limited to k <= column tile (B^T lower triangular)
  K_GE_J = 2,     // k >= column tile start (B lower triangular)
  K_LE_I = 3,     // k <= row tile (A lower triangular)
  K_GE_MAXIJ = 4  // k >= max(row tile, column tile) start (A^T A with A lower triangular)
};
enum TileMode {
  TILE_ALL = 0,
  TILE_LOWER = 1,         // only tiles with ti >= tj, only elements with i >= j are written
  TILE_LOWER_MIRROR = 2,  // tiles with ti >= tj, mirrored into the upper triangle
  TILE_LINEAR_GRID = 4    // flag set by the launcher: blockIdx.x enumerates the tiles with ti >= tj row by row
};

struct GemmParams {
  const float* A = nullptr;
  const float* B = nullptr;
  float* C = nullptr;
  float* const* C_list = nullptr;     // optional: per-batch output pointers (overrides C / sC)
  int64_t lda = 0, ldb = 0, ldc = 0;
  int64_t sA = 0, sB = 0, sC = 0;     // batch strides in elements
  int M = 0, N = 0, K = 0;
  int transA = 0, transB = 0;
  float alpha = 1.f, beta = 0.f;
  int kmode = 0, tile_mode = 0;
  const int* active = nullptr;        // optional per-batch flags: batch z runs only if active[z*active_stride] != 0
  int active_stride = 0;
  int split = 0;                      // 0: fp32 MFMA; 2 / 3: bf16 MFMA on operands split into that many bf16 pieces (gemm_x3.hpp)
  int chunked = 0;                    // non-zero: the contraction is summed in chunks (a fresh accumulator every 128 / 256 k, added
                                      // to a running total), which keeps the rounding error of a long sum near that of one
                                      // rounding instead of growing with the number of matrix instructions (fp32 kernel, and the
                                      // three-piece kernel for untransposed operands; ignored elsewhere)
  float scaleA = 1.f, scaleB = 1.f;   // fp16-piece variant only: powers of two the operands are multiplied by before the split
  float* absmax_out = nullptr;        // optional: the largest |C| of the result (of batch entry z: absmax_out[z * absmax_stride]) is
  int64_t absmax_stride = 0;          // folded into this word with an integer atomic maximum on its bit pattern (the caller
  int absmax_identity = 0;            // zeroes it first).  absmax_identity: the largest |C - I| instead, and a NaN in C ends up
                                      // in the word (as torch.max would return it) instead of being skipped
  float* C2 = nullptr;                // optional second result, same shape and batch layout as C with its own strides:
  int64_t ldc2 = 0, sC2 = 0;          // C2 = c2_scale * C + c2_diag * I (the next iterate's polynomial of a Newton iteration,
  float c2_scale = 0.f, c2_diag = 0.f;   // written while C is still in registers)
};

constexpr int GBT = 128, GBK = 16;     // GBT: granularity of the triangular contraction ranges (both tile sizes)
constexpr int G_KC_STRIDE = GBK + 4;    // [row][k] layout
template <int BT> struct GemmTile {
  static constexpr int IC_STRIDE = BT + 4;    // [k][row] layout
  static constexpr int PANEL = BT * G_KC_STRIDE > GBK * IC_STRIDE ? BT * G_KC_STRIDE : GBK * IC_STRIDE;
  static constexpr int CHUNKS = BT * GBK / 4 / 256;   // 16-byte chunks per thread per panel
};

// Loads this thread's two 16-byte chunks of a 128 x 16 operand panel.
//  kcontig: memory rows are the 128 tile rows, 16 k values contiguous.
//  else   : memory rows are the 16 k values, 128 tile rows contiguous.
template <int BT>
__device__ __forceinline__ void gemm_fetch(floatx4 (&reg)[GemmTile<BT>::CHUNKS], const float* __restrict__ P, int64_t ld,
                                           bool kcontig, int r0, int r_end, int k0, int k_end, bool vec_ok, int tid) {
  constexpr int RC = BT / 4;      // chunks per k-row in the [k][row] layout
#pragma unroll
  for (int u = 0; u < GemmTile<BT>::CHUNKS; ++u) {
    const int c = tid + 256 * u;
    int outer, inner, o_end, i_end;
    if (kcontig) { outer = r0 + (c >> 2); inner = k0 + 4 * (c & 3); o_end = r_end; i_end = k_end; }
    else { outer = k0 + c / RC; inner = r0 + 4 * (c % RC); o_end = k_end; i_end = r_end; }
    floatx4 v = {0.f, 0.f, 0.f, 0.f};
    if (outer < o_end && inner < i_end) {
      const float* src = P + static_cast<int64_t>(outer) * ld + inner;
      if (vec_ok && inner + 4 <= i_end) {
        v = *reinterpret_cast<const floatx4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (inner + e < i_end) v[e] = src[e];
      }
    }
    reg[u] = v;
  }
}

template <int BT>
__device__ __forceinline__ void gemm_stash(const floatx4 (&reg)[GemmTile<BT>::CHUNKS], float* __restrict__ lds,
                                           bool kcontig, int tid) {
  constexpr int RC = BT / 4;
#pragma unroll
  for (int u = 0; u < GemmTile<BT>::CHUNKS; ++u) {
    const int c = tid + 256 * u;
    const int off = kcontig ? (c >> 2) * G_KC_STRIDE + 4 * (c & 3) : (c / RC) * GemmTile<BT>::IC_STRIDE + 4 * (c % RC);
    *reinterpret_cast<floatx4*>(lds + off) = reg[u];
  }
}

// Reads the 8 k values (k = 8g + m) of tile row `row` for this lane.
template <int BT>
__device__ __forceinline__ void gemm_frag(float (&f)[8], const float* __restrict__ lds, bool kcontig, int row, int g) {
  if (kcontig) {
    const floatx4* q = reinterpret_cast<const floatx4*>(lds + row * G_KC_STRIDE + 8 * g);
    const floatx4 lo = q[0], hi = q[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) { f[e] = lo[e]; f[4 + e] = hi[e]; }
  } else {
#pragma unroll
    for (int m = 0; m < 8; ++m) f[m] = lds[(8 * g + m) * GemmTile<BT>::IC_STRIDE + row];
  }
}

// Running maximum of |v| (identity: of |v - 1| on the diagonal, |v| off it, and a NaN is kept once it has been seen).
__device__ __forceinline__ float gemm_fold_absmax(float vmax, float v, bool diagonal, int identity) {
  if (identity == 0) return fmaxf(vmax, fabsf(v));
  const float d = fabsf(v - (diagonal ? 1.f : 0.f));
  return (d > vmax || d != d) ? d : vmax;
}

// Folds a wave's maxima into the word at `out`.  Non-negative floats order like their bit patterns, and a NaN has a
// larger pattern than any number.
__device__ __forceinline__ void gemm_store_absmax(float* out, float vmax, int lane) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float other = __shfl_xor(vmax, o);
    vmax = (other > vmax || other != other) ? other : vmax;
  }
  vmax = fabsf(vmax);       // (a NaN of either sign: the pattern without the sign bit)
  if (lane == 0) atomicMax(reinterpret_cast<unsigned int*>(out), __builtin_bit_cast(unsigned int, vmax));
}

// One BT x BT tile (ti, tj) of batch entry z of the product described by p; lds: [2][2][PANEL] floats.
// CHUNKED: every 8 k-tiles (128 k) the accumulators are added to a running total and start again from zero: the
// matrix instruction rounds its accumulator once per two k, so a contraction over K rounds K/2 times at the full
// magnitude of the sum; in chunks, 64 roundings happen at the magnitude of one chunk and K/128 at the full one.
template <int TI, bool CHUNKED = false>
__device__ __forceinline__ void gemm_f32_tile(const GemmParams& p, int ti, int tj, int z,
                                              float (*lds)[2][GemmTile<64 * TI>::PANEL]) {
  constexpr int BT = 64 * TI;
  if (p.active != nullptr && p.active[static_cast<int64_t>(z) * p.active_stride] == 0) return;
  if (p.tile_mode != TILE_ALL && ti < tj) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1, g = lane >> 5, l32 = lane & 31;

  int kbeg = 0, kend = p.K;
  switch (p.kmode) {     // ranges rounded outwards to multiples of GBK; the operands are zero outside their triangle
    case K_LE_J: kend = min(p.K, (tj + 1) * BT); break;
    case K_GE_J: kbeg = tj * BT; break;
    case K_LE_I: kend = min(p.K, (ti + 1) * BT); break;
    case K_GE_MAXIJ: kbeg = max(ti, tj) * BT; break;
    default: break;
  }
  const float* __restrict__ A = p.A + static_cast<int64_t>(z) * p.sA;
  const float* __restrict__ B = p.B + static_cast<int64_t>(z) * p.sB;
  float* __restrict__ C = p.C_list != nullptr ? p.C_list[z] : p.C + static_cast<int64_t>(z) * p.sC;
  const bool a_kc = (p.transA == 0), b_kc = (p.transB != 0);
  const bool a_vec = (p.lda % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
  const bool b_vec = (p.ldb % 4 == 0) && ((reinterpret_cast<uintptr_t>(B) & 15) == 0);
  const int i0 = ti * BT, j0 = tj * BT;

  floatx16 acc[TI][TI];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TI; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  constexpr int TT = CHUNKED ? TI : 1;
  floatx16 tot[TT][TT];
  if constexpr (CHUNKED) {
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
      for (int b = 0; b < TI; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) tot[a][b][r] = 0.f;
  }

  const int nk = kbeg < kend ? (kend - kbeg + GBK - 1) / GBK : 0;
  floatx4 ra[GemmTile<BT>::CHUNKS], rb[GemmTile<BT>::CHUNKS];
  if (nk > 0) {
    gemm_fetch<BT>(ra, A, p.lda, a_kc, i0, p.M, kbeg, kend, a_vec, tid);
    gemm_fetch<BT>(rb, B, p.ldb, b_kc, j0, p.N, kbeg, kend, b_vec, tid);
    gemm_stash<BT>(ra, lds[0][0], a_kc, tid);
    gemm_stash<BT>(rb, lds[0][1], b_kc, tid);
  }
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) {
      const int k0 = kbeg + (kt + 1) * GBK;
      gemm_fetch<BT>(ra, A, p.lda, a_kc, i0, p.M, k0, kend, a_vec, tid);
      gemm_fetch<BT>(rb, B, p.ldb, b_kc, j0, p.N, k0, kend, b_vec, tid);
    }
    float fa[TI][8], fb[TI][8];
#pragma unroll
    for (int a = 0; a < TI; ++a) gemm_frag<BT>(fa[a], lds[buf][0], a_kc, 32 * TI * wr + 32 * a + l32, g);
#pragma unroll
    for (int b = 0; b < TI; ++b) gemm_frag<BT>(fb[b], lds[buf][1], b_kc, 32 * TI * wc + 32 * b + l32, g);
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
      for (int a = 0; a < TI; ++a)
#pragma unroll
        for (int b = 0; b < TI; ++b) acc[a][b] = mfma_f32(fa[a][m], fb[b][m], acc[a][b]);
    if constexpr (CHUNKED) {
      if ((kt & 7) == 7) {
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
          for (int b = 0; b < TI; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) { tot[a][b][r] += acc[a][b][r]; acc[a][b][r] = 0.f; }
      }
    }
    if (kt + 1 < nk) {
      gemm_stash<BT>(ra, lds[buf ^ 1][0], a_kc, tid);
      gemm_stash<BT>(rb, lds[buf ^ 1][1], b_kc, tid);
    }
    __syncthreads();
  }

  if constexpr (CHUNKED) {
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
      for (int b = 0; b < TI; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] += tot[a][b][r];
  }
  const bool lower_only = (p.tile_mode == TILE_LOWER);
  const bool mirror = (p.tile_mode == TILE_LOWER_MIRROR) && (ti != tj);
  float* __restrict__ C2 = p.C2 != nullptr ? p.C2 + static_cast<int64_t>(z) * p.sC2 : nullptr;
  float vmax = 0.f;
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TI; ++b) {
      const int gj = j0 + 32 * TI * wc + 32 * b + l32;
      if (gj >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gi = i0 + 32 * TI * wr + 32 * a + 8 * (r >> 2) + 4 * g + (r & 3);
        if (gi >= p.M) continue;
        if (lower_only && gi < gj) continue;
        float v = p.alpha * acc[a][b][r];
        float* dst = C + static_cast<int64_t>(gi) * p.ldc + gj;
        if (p.beta != 0.f) v += p.beta * *dst;
        *dst = v;
        if (mirror) C[static_cast<int64_t>(gj) * p.ldc + gi] = v;
        vmax = gemm_fold_absmax(vmax, v, gi == gj, p.absmax_identity);
        if (C2 != nullptr) {
          const float w = p.c2_scale * v + (gi == gj ? p.c2_diag : 0.f);
          C2[static_cast<int64_t>(gi) * p.ldc2 + gj] = w;
          if (mirror) C2[static_cast<int64_t>(gj) * p.ldc2 + gi] = w;
        }
      }
    }
  if (p.absmax_out != nullptr) gemm_store_absmax(p.absmax_out + static_cast<int64_t>(z) * p.absmax_stride, vmax, lane);
}

template <int TI, bool CHUNKED = false>
static __global__ __launch_bounds__(256) void gemm_f32_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(16))) float lds[2][2][GemmTile<64 * TI>::PANEL];
  gemm_f32_tile<TI, CHUNKED>(p, blockIdx.y, blockIdx.x, blockIdx.z, lds);
}

}  // namespace ak

#include "gemm_x3.hpp"

namespace ak {

// Constants of the product library; variables that a setter can change only in tuning builds (-DAK_TUNING_HOOKS).
#ifdef AK_TUNING_HOOKS
inline int g_x3_double_buffer = 1;
inline int g_x3_min_groups = 100, g_x3_min_k = 256;
#else
constexpr int g_x3_double_buffer = 1;
constexpr int g_x3_min_groups = 100, g_x3_min_k = 256;
#endif

inline int launch_gemm(const GemmParams& p, int batch, hipStream_t stream) {
  if (p.M <= 0 || p.N <= 0 || batch <= 0) return AK_OK;
  const int64_t tiles128 = static_cast<int64_t>((p.N + 127) / 128) * ((p.M + 127) / 128) * batch;
  const bool lower = p.tile_mode != TILE_ALL;
  const int64_t work_groups = lower ? tiles128 / 2 : tiles128;
  // The split kernel (128 x 128 tiles, a pipeline that needs a few k-tiles to fill) pays off once its tiles
  // fill most of the device; below that the 64 x 64 tiles of the fp32 kernel spread the work better.
  if (p.split >= 2 && work_groups >= g_x3_min_groups && p.K >= g_x3_min_k && gemm_x3_ok(p)) {
    dim3 grid((p.N + 127) / 128, (p.M + 127) / 128, batch);
    GemmParams q = p;
    if (lower && p.M == p.N) {                  // square result, lower tiles only: enumerate just those
      const unsigned T = grid.x;
      grid = dim3(T * (T + 1) / 2, 1, batch);
      q.tile_mode |= TILE_LINEAR_GRID;
    }
    // three pieces: the double-buffered loop (one work group per CU, MFMAs and split arithmetic interleaved by
    // hand), one instantiation per pair of operand layouts; two pieces: the single-buffered loop
    if (p.split == 3 && g_x3_double_buffer) {
      if (p.transA == 0 && p.transB != 0) hipLaunchKernelGGL((gemm_x3_kernel<3, true, 1, 1>), grid, dim3(256), 0, stream, q);
      else if (p.transA == 0 && p.chunked) hipLaunchKernelGGL((gemm_x3_kernel<3, true, 1, 0, true>), grid, dim3(256), 0, stream, q);
      else if (p.transA == 0) hipLaunchKernelGGL((gemm_x3_kernel<3, true, 1, 0>), grid, dim3(256), 0, stream, q);
      else if (p.transB != 0) hipLaunchKernelGGL((gemm_x3_kernel<3, true, 0, 1>), grid, dim3(256), 0, stream, q);
      else hipLaunchKernelGGL((gemm_x3_kernel<3, true, 0, 0>), grid, dim3(256), 0, stream, q);
    } else if (p.split == 2) {
      hipLaunchKernelGGL((gemm_x3_kernel<2, false>), grid, dim3(256), 0, stream, q);
    } else {
      hipLaunchKernelGGL((gemm_x3_kernel<3, false>), grid, dim3(256), 0, stream, q);
    }
    return check_launch();
  }
  // 128 x 128 tiles when they alone fill the 256 CUs twice over, else 64 x 64 tiles (four times the work groups)
  if (work_groups >= 512) {
    dim3 grid((p.N + 127) / 128, (p.M + 127) / 128, batch);
    if (p.chunked) hipLaunchKernelGGL((gemm_f32_kernel<2, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gemm_f32_kernel<2>, grid, dim3(256), 0, stream, p);
  } else {
    dim3 grid((p.N + 63) / 64, (p.M + 63) / 64, batch);
    if (p.chunked) hipLaunchKernelGGL((gemm_f32_kernel<1, true>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gemm_f32_kernel<1>, grid, dim3(256), 0, stream, p);
  }
  return check_launch();
}

inline GemmParams make_gemm(int transA, int transB, int M, int N, int K, float alpha, const float* A, int64_t lda,
                            const float* B, int64_t ldb, float beta, float* C, int64_t ldc) {
  GemmParams p;
  p.A = A; p.B = B; p.C = C;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.M = M; p.N = N; p.K = K;
  p.transA = transA; p.transB = transB;
  p.alpha = alpha; p.beta = beta;
  p.kmode = K_FULL; p.tile_mode = TILE_ALL;
  return p;
}

}  // namespace ak
