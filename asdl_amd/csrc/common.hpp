// Shared device helpers for the gfx950 kernels: MFMA fragment types, the layout of a 32x32
// accumulator tile, LDS transpose reads, and the symmetric epilogue used by both SYRK kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/asdl_amd.h"

namespace ak {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

// v_mfma_f32_32x32x16_bf16: lane l feeds A[i = l%32][k = 8*(l/32) + e] and B[k][j = l%32],
// e = 0..7; accumulator register r of lane l is C[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32].
__device__ __forceinline__ floatx16 mfma_bf16(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
// v_mfma_f32_32x32x2_f32: lane l feeds A[i = l%32][k = l/32] and B[k = l/32][j = l%32];
// same accumulator layout.
__device__ __forceinline__ floatx16 mfma_f32(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane j receives element (j % 4) of the
// 8 bytes addressed by lanes 4e + j/4, e = 0..3.  With lanes 4e..4e+3 pointing at row k0+e of a
// [k][i] tile (16 consecutive i), lane j ends up with column i0 + j for k0..k0+3.
__device__ __forceinline__ short4v lds_read_tr16(const void* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (short4v __attribute__((address_space(3)))*)(p));
}

__device__ __forceinline__ bf16x8 pack_bf16x8(short4v lo, short4v hi) {
  short8v v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

// Lower-triangular tile enumeration: linear id -> (ti, tj), tj <= ti, row by row (id = ti (ti + 1) / 2 + tj).
__device__ __forceinline__ void decode_lower_tile(int id, int& ti, int& tj) {
  int row = static_cast<int>((__builtin_sqrtf(8.f * static_cast<float>(id) + 1.f) - 1.f) * 0.5f);
  while (row * (row + 1) / 2 > id) --row;
  while ((row + 1) * (row + 2) / 2 <= id) ++row;
  ti = row;
  tj = id - row * (row + 1) / 2;
}

// Upper-triangular tile enumeration: linear id -> (ti, tj), ti <= tj < T, row-major.
__device__ __forceinline__ void decode_upper_tile(int id, int T, int& ti, int& tj) {
  int row = 0, len = T;
  while (id >= len) { id -= len; ++row; --len; }
  ti = row;
  tj = row + id;
}

// The SYRK epilogues read the old result (beta != 0) through a 32-bit buffer descriptor: results of 4 GiB and more
// cannot be accumulated into.
// (d + 31: the 32-bit offsets of a partial last block row are formed for rows up to d + 30 before the range check.)
inline bool syrk_beta_ok(float beta, int64_t d, int64_t ldc) {
  return beta == 0.f || ((d + 31) * ldc + d) * 4 < 0xFFFFFF00ll;
}

// Symmetric epilogue for one wave's accumulators of a BT x BT output tile at (ti, tj), ti <= tj.
// acc[a][b] is the 32x32 MFMA tile at rows row0 + 32a, cols col0 + 32b of the WG tile.
// Writes C[i][j] = beta*C[i][j] + alpha*acc and, off the diagonal tile, the mirror C[j][i].
template <int TI, int TJ>
__device__ __forceinline__ void syrk_epilogue(floatx16 (&acc)[TI][TJ], float* __restrict__ C, int64_t ldc,
                                              int64_t d, int64_t gi0, int64_t gj0, bool diag_tile,
                                              float alpha, float beta, int lane) {
  const int g = lane >> 5, l32 = lane & 31;
  const bool vec_mirror = (ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(C) & 15) == 0);
  // Phase 1: acc <- alpha * acc (+ beta * C).  All reads of C come before the first store: the compiler cannot
  // prove that a store to C leaves a later read alone, so reads that follow stores are issued one memory latency
  // after another.  The reads go through a buffer descriptor of C: one 32-bit offset register per 32 x 32 block and
  // lane, the row within the block as a scalar offset (a load under a per-element condition gets a wait of its
  // own: 16 * TI * TJ memory latencies in a row; 64-bit addresses and clamped indices for as many loads in flight
  // cost more registers than the widest tile has).  The hardware checks only the vector offset plus the
  // instruction's immediate against the descriptor's size; the scalar offset is added to the address afterwards,
  // unchecked.  So the scalar row offset is used only in 32-row blocks that lie wholly inside the matrix (a test
  // that is uniform over the wave); the one partial block row of a matrix with d % 32 != 0 puts the row into the
  // vector offset, where rows beyond the matrix are out of range and read as zero.  Lanes of columns beyond d get
  // an out-of-range vector offset for the same reason (their accumulators are never stored).
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] *= alpha;
  if (beta != 0.f) {
    // (the entry points refuse beta != 0 for a result of 4 GiB and more: syrk_beta_ok)
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(C, 0, static_cast<int>(((d - 1) * ldc + d) * 4), 0x00020000);
    const uint32_t ldc4 = static_cast<uint32_t>(ldc) * 4u;
#pragma unroll
    for (int a = 0; a < TI; ++a) {
#pragma unroll
      for (int b = 0; b < TJ; ++b) {
        // a lane whose column lies beyond the matrix gets an offset that is out of range whatever the row
        const bool col_ok = gj0 + 32 * b + l32 < d;
        const uint32_t voff = static_cast<uint32_t>(gi0 + 32 * a + 4 * g) * ldc4 +
                              static_cast<uint32_t>(gj0 + 32 * b + l32) * 4u;
        if (gi0 + 32 * a + 32 <= d) {
          const uint32_t vsel = col_ok ? voff : 0xFFFFFF00u;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float c = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, vsel, (8 * (r >> 2) + (r & 3)) * ldc4, 0));
            acc[a][b][r] += beta * c;
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const uint32_t vrow = voff + (8 * (r >> 2) + (r & 3)) * ldc4;
            const float c = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, col_ok ? vrow : 0xFFFFFF00u, 0, 0));
            acc[a][b][r] += beta * c;
          }
        }
      }
    }
  }
  // Phase 2: the tile and, off the diagonal, its mirror image.
#pragma unroll
  for (int a = 0; a < TI; ++a) {
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      const int64_t gj = gj0 + 32 * b + l32;
      if (gj >= d) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t gi = gi0 + 32 * a + 8 * q + 4 * g;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (gi + e < d) C[(gi + e) * ldc + gj] = acc[a][b][4 * q + e];
        if (!diag_tile) {
          if (vec_mirror && gi + 3 < d) {
            floatx4 w = {acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]};
            *reinterpret_cast<floatx4*>(C + gj * ldc + gi) = w;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (gi + e < d) C[gj * ldc + gi + e] = acc[a][b][4 * q + e];
          }
        }
      }
    }
  }
}

// Split-K partial tile store / load in accumulator order: [(a,b,q)][thread] float4, coalesced.
template <int TI, int TJ>
__device__ __forceinline__ void store_partial(floatx16 (&acc)[TI][TJ], float* __restrict__ wsTile, int tid) {
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        floatx4 w = {acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]};
        reinterpret_cast<floatx4*>(wsTile)[((a * TJ + b) * 4 + q) * 256 + tid] = w;
      }
}

template <int TI, int TJ>
__device__ __forceinline__ void add_partial(floatx16 (&acc)[TI][TJ], const float* __restrict__ wsTile, int tid) {
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        floatx4 w = reinterpret_cast<const floatx4*>(wsTile)[((a * TJ + b) * 4 + q) * 256 + tid];
        acc[a][b][4 * q] += w[0];
        acc[a][b][4 * q + 1] += w[1];
        acc[a][b][4 * q + 2] += w[2];
        acc[a][b][4 * q + 3] += w[3];
      }
}

// Sums the split-K partials and applies the symmetric epilogue.  grid (upper tiles, TI*TJ*4): each work
// group owns one float4 slot (a, b, q) of every thread's accumulators, so a tile is reduced by 4*TI*TJ work
// groups in parallel; the sum over splits runs in a fixed order (deterministic).
template <int TI, int TJ>
__global__ __launch_bounds__(256) void syrk_finalize_kernel(const float* __restrict__ ws, int nsplit, int T,
                                                            float* __restrict__ C, int64_t ldc, int64_t d,
                                                            float alpha, float beta) {
  constexpr int BT = 64 * TI;
  static_assert(TI == TJ, "square tiles");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1, g = lane >> 5, l32 = lane & 31;
  int ti, tj;
  decode_upper_tile(blockIdx.x, T, ti, tj);
  const int ntiles = gridDim.x;
  const int slot = blockIdx.y;                 // (a * TJ + b) * 4 + q
  const int q = slot & 3, b = (slot >> 2) % TJ, a = (slot >> 2) / TJ;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  const floatx4* src = reinterpret_cast<const floatx4*>(ws) + (static_cast<size_t>(blockIdx.x) * (BT * BT / 4)) +
                       slot * 256 + tid;
  const size_t split_stride = static_cast<size_t>(ntiles) * (BT * BT / 4);
  for (int s = 0; s < nsplit; ++s) {
    const floatx4 w = src[s * split_stride];
    acc[0] += w[0]; acc[1] += w[1]; acc[2] += w[2]; acc[3] += w[3];
  }
  const int64_t gj = static_cast<int64_t>(tj) * BT + 32 * TJ * wc + 32 * b + l32;
  const int64_t gi = static_cast<int64_t>(ti) * BT + 32 * TI * wr + 32 * a + 8 * q + 4 * g;
  if (gj >= d) return;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float x = alpha * acc[e];
    if (beta != 0.f && gi + e < d) x += beta * C[(gi + e) * ldc + gj];
    v[e] = x;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (gi + e < d) C[(gi + e) * ldc + gj] = v[e];
  if (ti != tj) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (gi + e < d) C[gj * ldc + gi + e] = v[e];
  }
}

// Division by a run-time constant: q = umulhi(x, ceil(2^32 / d)), exact while x * d < 2^32.
__host__ __device__ inline uint32_t make_magic(uint32_t d) { return static_cast<uint32_t>((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ uint32_t fastdiv(uint32_t x, uint32_t magic, uint32_t d) {
  return d == 1 ? x : __umulhi(x, magic);
}

// bf16 X^T X with direct global -> LDS panel loads (syrk_dtl.hip).  *_ok tells whether the operand meets its
// alignment and range requirements; the launcher may still answer AK_ERR_UNSUPPORTED / AK_ERR_WORKSPACE, on
// which callers take the register-staged kernel.
bool syrk_dtl_plain_ok(const void* X, int64_t M, int64_t d, int64_t ldx);
size_t syrk_dtl_plain_ws_bytes(int64_t M, int64_t d, int64_t ldx);
int syrk_dtl_plain(const void* X, int64_t M, int64_t d, int64_t ldx, float alpha, float beta, float* C, int64_t ldc,
                   void* ws, size_t ws_bytes, hipStream_t stream);

// Input factor of a convolution with d = C*kh*kw <= 160 from an LDS-resident input window (conv_patch.hip); x has
// element strides (sn, sc, sh_el, sw_el).  The workspace query answers 0, the launcher AK_ERR_UNSUPPORTED, for
// other layers.
size_t conv_patch_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw);
int conv_patch_syrk(const void* x, int dtype, int64_t sn, int64_t sc, int64_t sh_el, int64_t sw_el, int64_t N, int64_t C,
                    int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw, float alpha, float beta,
                    float* A, int64_t lda, void* ws, size_t ws_bytes, hipStream_t stream);

// Input factor of a 3 x 3 / stride 1 / padding 1 convolution on a channels-last bf16 input with a multiple of 64
// channels, from shifted correlations of the input (conv_corr.hip).  The workspace query answers 0, the launcher
// AK_ERR_UNSUPPORTED, for other layers.
size_t conv_corr_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw);
int conv_corr_syrk(const void* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                   int pw, float alpha, float beta, float* A, int64_t lda, void* ws, size_t ws_bytes, hipStream_t stream);

// The same for an fp32 NCHW input: split into three bf16 planes first (products at the accuracy of fp32).
size_t conv_corr_f32_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw);
int conv_corr_syrk_f32(const float* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                       int pw, float alpha, float beta, float* A, int64_t lda, void* ws, size_t ws_bytes,
                       hipStream_t stream);

inline int check_launch() { return hipGetLastError() == hipSuccess ? AK_OK : AK_ERR_LAUNCH; }

// Split-K factor shared by the SYRK front ends: enough work groups to fill 256 CUs twice over
// while every split still runs a useful number of k-steps.
inline int pick_nsplit(int64_t ntiles, int64_t ksteps) {
  int64_t want = (512 + ntiles - 1) / ntiles;
  int64_t cap = ksteps / 8;
  if (cap < 1) cap = 1;
  int64_t s = want < cap ? want : cap;
  if (s > 256) s = 256;
  if (s < 1) s = 1;
  return static_cast<int>(s);
}

}  // namespace ak
