// fp32 GEMM on the bf16 matrix cores: every fp32 operand element is split exactly into three bf16 pieces
// (hi = x rounded to the nearest bf16, mid = x - hi rounded, lo = x - hi - mid, which needs no rounding any more:
// hi + mid + lo == x), and the product is accumulated in fp32 from the six piece products that matter:
//   x*y ~= hi*hi' + hi*mid' + mid*hi' + hi*lo' + lo*hi' + mid*mid'      (dropped terms are below 2^-24 |x y|),
// i.e. the accuracy of an fp32 multiply at 6/16 of the cost of the fp32 MFMA.  With NSPLIT = 2 only hi and mid
// are kept (16 mantissa bits, 3 products) for callers whose tolerance allows it.  Rounding to nearest (one packed
// hardware conversion per two elements) leaves errors of either sign; cutting the pieces off instead would bias
// every product towards zero, which a sum of squares (a Gram matrix) accumulates coherently.
//
// Same interface as gemm_f32_kernel (GemmParams: transposes, triangular contraction ranges, lower-triangle tile
// modes, batches).  One work group = 4 waves (2x2) = one 128x128 tile, k-tiles of 32.  An operand whose contraction
// index is contiguous in memory is kept in the LDS as [row][32 k] with the 16-byte chunks of a row XOR-swizzled by
// (row/4)%4, so that the ds_read_b128 of 16 consecutive rows hits 64 different banks; one whose row/column index
// is contiguous is kept as [32 columns][32 k-rows][64 B] blocks and read with ds_read_b64_tr_b16 (no bank
// conflicts, no transposed copies).
//
// Two main loops.  Single-buffered (two work groups per CU, which overlap each other): the fp32 panels are fetched
// into registers one k-tile ahead, split and written to the LDS after the MFMAs of the current k-tile, two
// barriers per k-tile.  Double-buffered (DB, 96 KB of LDS, one work group per CU): one barrier per k-tile and a
// fixed instruction order in which every MFMA is followed by a sixth of the split of one float4 of the next
// k-tile, so that the vector ALU works in the shadow of the matrix pipe; the operand layouts are template
// parameters there, which makes the loop body a single basic block.  Measured on 4096^3: 776 -> 697 us, on
// 2048^3 (one tile per CU) 150 -> 96 us.
#pragma once
#include <type_traits>
#include "common.hpp"

namespace ak {

#define AK_LDS3 __attribute__((address_space(3)))
typedef uint32_t x3_u32x2 __attribute__((ext_vector_type(2)));
typedef float x3_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 x3_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 x3_f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 x3_f16x8 __attribute__((ext_vector_type(8)));

// One matrix instruction on 16-byte fragments that hold bf16 pieces, or (HALF) fp16 pieces.
template <bool HALF>
__device__ __forceinline__ floatx16 x3_mfma(bf16x8 a, bf16x8 b, floatx16 c) {
  if constexpr (HALF)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(x3_f16x8, a), __builtin_bit_cast(x3_f16x8, b), c, 0, 0, 0);
  else
    return mfma_bf16(a, b, c);
}

constexpr int X3_BT = 128, X3_BK = 32;
constexpr int X3_PLANE = X3_BT * X3_BK * 2;      // bytes of one bf16 plane of one operand panel

struct X3Fetch {
  floatx4 v[4];
};

// Loads this thread's four float4 of a 128 x 32 operand panel.  kcontig: memory rows are the 128 tile rows and
// hold 32 consecutive k; else memory rows are the 32 k values and hold 128 consecutive tile rows.
template <bool INTERIOR>
__device__ __forceinline__ void x3_fetch(X3Fetch& r, const float* __restrict__ P, int64_t ld, bool kcontig, int r0,
                                         int r_end, int k0, int k_end, int tid) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int f = tid + 256 * u;
    int outer, inner, o_end, i_end;
    if (kcontig) { outer = r0 + (f >> 3); inner = k0 + 4 * (f & 7); o_end = r_end; i_end = k_end; }
    else { outer = k0 + (f >> 5); inner = r0 + 4 * (f & 31); o_end = k_end; i_end = r_end; }
    if (INTERIOR) {
      r.v[u] = *reinterpret_cast<const floatx4*>(P + static_cast<int64_t>(outer) * ld + inner);
    } else {
      // no branch around the load: an invalid chunk reads the first chunk of the matrix and is zeroed afterwards
      const bool ok = outer < o_end && inner < i_end;        // inner and i_end are multiples of 4
      const float* src = ok ? P + static_cast<int64_t>(outer) * ld + inner : P;
      const floatx4 w = *reinterpret_cast<const floatx4*>(src);
      const floatx4 z = {0.f, 0.f, 0.f, 0.f};
      r.v[u] = ok ? w : z;
    }
  }
}

// One of this thread's four float4 of a panel (chunk u of x3_fetch).
template <bool INTERIOR>
__device__ __forceinline__ floatx4 x3_fetch_one(const float* __restrict__ P, int64_t ld, bool kcontig, int r0, int r_end,
                                                int k0, int k_end, int tid, int u) {
  const int f = tid + 256 * u;
  int outer, inner, o_end, i_end;
  if (kcontig) { outer = r0 + (f >> 3); inner = k0 + 4 * (f & 7); o_end = r_end; i_end = k_end; }
  else { outer = k0 + (f >> 5); inner = r0 + 4 * (f & 31); o_end = k_end; i_end = r_end; }
  if (INTERIOR) return *reinterpret_cast<const floatx4*>(P + static_cast<int64_t>(outer) * ld + inner);
  const bool ok = outer < o_end && inner < i_end;
  const float* src = ok ? P + static_cast<int64_t>(outer) * ld + inner : P;
  const floatx4 w = *reinterpret_cast<const floatx4*>(src);
  const floatx4 z = {0.f, 0.f, 0.f, 0.f};
  return ok ? w : z;
}

// Byte offset of chunk u inside a plane (the layouts of x3_stash).
__device__ __forceinline__ uint32_t x3_chunk_offset(bool kcontig, int tid, int u) {
  const int f = tid + 256 * u;
  if (kcontig) {
    const int row = f >> 3, c4 = f & 7;
    return row * 64 + 16 * ((c4 >> 1) ^ ((row >> 2) & 3)) + 8 * (c4 & 1);
  }
  const int krow = f >> 5, c4 = f & 31;
  return (c4 >> 3) * 2048 + krow * 64 + (c4 & 7) * 8;
}

// Splits the fetched panel into NSPLIT bf16 planes and writes them to the LDS.  HALF: fp16 pieces of scale * x
// instead (11 significant bits each: two pieces carry 22 bits; `scale`, a power of two, brings the operand into the
// range of fp16: the caller guarantees |scale * x| <= 2^15 and divides the result by the scales of both operands).
template <int NSPLIT, bool HALF = false>
__device__ __forceinline__ void x3_stash(const X3Fetch& r, AK_LDS3 unsigned char* panel, bool kcontig, int tid,
                                         float scale = 1.f) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int f = tid + 256 * u;
    uint32_t off;
    if (kcontig) {
      const int row = f >> 3, c4 = f & 7;
      off = row * 64 + 16 * ((c4 >> 1) ^ ((row >> 2) & 3)) + 8 * (c4 & 1);
    } else {
      const int krow = f >> 5, c4 = f & 31;
      off = (c4 >> 3) * 2048 + krow * 64 + (c4 & 7) * 8;
    }
    // Every piece is the remainder rounded to the nearest bf16 (one packed conversion per pair of elements);
    // x - hi and x - hi - mid are exact in fp32, and what is left after two pieces has at most 8 significant
    // bits, so the third piece is exact: hi + mid + lo == x.
    uint32_t pair[NSPLIT][2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      x3_f32x2 rem = {r.v[u][2 * e], r.v[u][2 * e + 1]};
      if constexpr (HALF) rem *= scale;
#pragma unroll
      for (int s = 0; s < NSPLIT; ++s) {
        if constexpr (HALF) {
          const x3_f16x2 h = __builtin_convertvector(rem, x3_f16x2);
          pair[s][e] = __builtin_bit_cast(uint32_t, h);
          if (s + 1 < NSPLIT) rem -= __builtin_convertvector(h, x3_f32x2);
        } else {
          const x3_bf16x2 h = __builtin_convertvector(rem, x3_bf16x2);
          pair[s][e] = __builtin_bit_cast(uint32_t, h);
          if (s + 1 < NSPLIT) rem -= __builtin_convertvector(h, x3_f32x2);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < NSPLIT; ++s) {
      x3_u32x2 w;
      w[0] = pair[s][0];
      w[1] = pair[s][1];
      *reinterpret_cast<AK_LDS3 x3_u32x2*>(panel + s * X3_PLANE + off) = w;
    }
  }
}

// The 8 k values (16*h + 8*g ...) of tile row `row` for this lane, as an MFMA operand.
__device__ __forceinline__ bf16x8 x3_frag(AK_LDS3 const unsigned char* plane, bool kcontig, int row, int h, int lane) {
  if (kcontig) {
    const int g = lane >> 5;
    return *reinterpret_cast<AK_LDS3 const bf16x8*>(plane + row * 64 + 16 * ((2 * h + g) ^ ((row >> 2) & 3)));
  }
  // row = 32*cb + (lane % 32): the transposing read serves 16 columns per half-wave group
  const int g = lane >> 5, hl = (lane >> 4) & 1, j16 = lane & 15;
  AK_LDS3 const unsigned char* q = plane + (row >> 5) * 2048 + (16 * h + 8 * g + (j16 >> 2)) * 64 + hl * 32 + (j16 & 3) * 8;
  const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AK_LDS3 short4v*)(q));
  const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((AK_LDS3 short4v*)(q + 256));
  return pack_bf16x8(lo, hi);
}

// One 128 x 128 tile (ti, tj) of batch entry z of the product described by p.
// CHUNKED: the products of the leading pieces, which carry the magnitude of the result, have an
// accumulator of their own that is added to a running total every 8 k-tiles (256 k: 16 roundings at the magnitude of
// a chunk, K/256 at the full one); the five cross products of three pieces, 2^-8 and less of that magnitude, share a
// second one (with two pieces the two cross products stay with the leading one: a third set of accumulators would
// halve the work groups per CU).
// The sum then carries about one rounding error instead of one that grows with 6 K / 16 accumulator roundings.
template <int NSPLIT, bool DB, int AKC = -1, int BKC = -1, bool HALF = false, bool CHUNKED = false>
__device__ __forceinline__ void gemm_x3_tile(const GemmParams& p, int ti, int tj, int z, AK_LDS3 unsigned char* lds) {
  static_assert(!HALF || (NSPLIT == 2 && !DB), "fp16 pieces: two of them, single-buffered loop");
  static_assert(!CHUNKED || NSPLIT >= 2, "chunked sums: split operands");
  constexpr int BT = X3_BT, BK = X3_BK;
  constexpr int BUF = 2 * NSPLIT * X3_PLANE;        // both operands' planes of one k-tile
  AK_LDS3 unsigned char* panelA = lds;
  AK_LDS3 unsigned char* panelB = lds + NSPLIT * X3_PLANE;
  if (p.active != nullptr && p.active[static_cast<int64_t>(z) * p.active_stride] == 0) return;
  if (p.tile_mode != TILE_ALL && ti < tj) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1, g = lane >> 5, l32 = lane & 31;

  int kbeg = 0, kend = p.K;
  switch (p.kmode) {     // ranges rounded outwards to multiples of the tile; the operands are zero outside their triangle
    case K_LE_J: kend = min(p.K, (tj + 1) * BT); break;
    case K_GE_J: kbeg = tj * BT; break;
    case K_LE_I: kend = min(p.K, (ti + 1) * BT); break;
    case K_GE_MAXIJ: kbeg = max(ti, tj) * BT; break;
    default: break;
  }
  const float* __restrict__ A = p.A + static_cast<int64_t>(z) * p.sA;
  const float* __restrict__ B = p.B + static_cast<int64_t>(z) * p.sB;
  float* __restrict__ C = p.C_list != nullptr ? p.C_list[z] : p.C + static_cast<int64_t>(z) * p.sC;
  // operand layouts: fixed at compile time where the caller knows them (one basic block per loop body then)
  const bool a_kc = AKC < 0 ? (p.transA == 0) : (AKC != 0), b_kc = BKC < 0 ? (p.transB != 0) : (BKC != 0);
  const int i0 = ti * BT, j0 = tj * BT;

  floatx16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  constexpr int TT = CHUNKED ? 2 : 1, TS = (CHUNKED && NSPLIT >= 3) ? 2 : 1;
  floatx16 small[TS][TS], tot[TT][TT];
  if constexpr (CHUNKED) {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          tot[a][b][r] = 0.f;
          if constexpr (NSPLIT >= 3) small[a][b][r] = 0.f;
        }
  }
  // end of k-tile kt: every eighth one moves the leading products' accumulators into the running total
  auto end_of_ktile = [&](int kt) {
    if constexpr (CHUNKED) {
      if ((kt & 7) == 7) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) { tot[a][b][r] += acc[a][b][r]; acc[a][b][r] = 0.f; }
      }
    }
  };

  const int nk = kbeg < kend ? (kend - kbeg + BK - 1) / BK : 0;
  const bool interior = i0 + BT <= p.M && j0 + BT <= p.N && (kend - kbeg) % BK == 0;

  // The MFMAs of one k-tile, operands read from the planes at `buf`.
  auto multiply = [&](AK_LDS3 unsigned char* buf) {
    AK_LDS3 unsigned char* pa = buf;
    AK_LDS3 unsigned char* pb = buf + NSPLIT * X3_PLANE;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      bf16x8 fa[2][NSPLIT], fb[2][NSPLIT];
#pragma unroll
      for (int s = 0; s < NSPLIT; ++s) {
#pragma unroll
        for (int a = 0; a < 2; ++a) fa[a][s] = x3_frag(pa + s * X3_PLANE, a_kc, 64 * wr + 32 * a + l32, h, lane);
#pragma unroll
        for (int b = 0; b < 2; ++b) fb[b][s] = x3_frag(pb + s * X3_PLANE, b_kc, 64 * wc + 32 * b + l32, h, lane);
      }
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          // smallest terms first
          if constexpr (CHUNKED && NSPLIT >= 3) {
            small[a][b] = x3_mfma<HALF>(fa[a][1], fb[b][1], small[a][b]);
            small[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][2], small[a][b]);
            small[a][b] = x3_mfma<HALF>(fa[a][2], fb[b][0], small[a][b]);
            small[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][1], small[a][b]);
            small[a][b] = x3_mfma<HALF>(fa[a][1], fb[b][0], small[a][b]);
            acc[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][0], acc[a][b]);
            continue;
          }
          if constexpr (NSPLIT >= 3) {
            acc[a][b] = x3_mfma<HALF>(fa[a][1], fb[b][1], acc[a][b]);
            acc[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][2], acc[a][b]);
            acc[a][b] = x3_mfma<HALF>(fa[a][2], fb[b][0], acc[a][b]);
          }
          if constexpr (NSPLIT >= 2) {
            acc[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][1], acc[a][b]);
            acc[a][b] = x3_mfma<HALF>(fa[a][1], fb[b][0], acc[a][b]);
          }
          acc[a][b] = x3_mfma<HALF>(fa[a][0], fb[b][0], acc[a][b]);
        }
    }
  };

  auto mainloop = [&](auto interior_tag) {
    constexpr bool INTERIOR = decltype(interior_tag)::value;
    X3Fetch ra, rb;
    auto fetch = [&](int kt) {
      const int k0 = kbeg + kt * BK;
      x3_fetch<INTERIOR>(ra, A, p.lda, a_kc, i0, p.M, k0, kend, tid);
      x3_fetch<INTERIOR>(rb, B, p.ldb, b_kc, j0, p.N, k0, kend, tid);
    };
    auto stash = [&](AK_LDS3 unsigned char* buf) {
      x3_stash<NSPLIT, HALF>(ra, buf, a_kc, tid, p.scaleA);
      x3_stash<NSPLIT, HALF>(rb, buf + NSPLIT * X3_PLANE, b_kc, tid, p.scaleB);
    };
    if (nk > 0) {
      fetch(0);
      stash(lds);
    }
    if constexpr (DB) {
      // Two LDS buffers, one barrier per k-tile: the split and store of k-tile kt+1 (into the other buffer) and
      // the global loads of k-tile kt+2 are issued ahead of the MFMAs of k-tile kt, in whose shadow they run.
      if (nk > 1) fetch(1);
      __syncthreads();
      int kt = 0;
      if constexpr (NSPLIT == 3 && AKC >= 0 && BKC >= 0) {
        // Fixed instruction order, one matrix instruction at a time: MFMA m of this k-tile, then one sixth of
        // the split of one float4 of the next k-tile (a packed conversion, two unpacks, two subtractions: about
        // as many cycles as the MFMA keeps the matrix pipe busy); after the sixth sixth the three LDS stores of
        // that float4 and the global load that refills its registers from the k-tile after next.  48 MFMAs, 48
        // sixths (8 float4 per thread x 3 pieces x 2 pairs).
        uint32_t offA[4], offB[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { offA[u] = x3_chunk_offset(a_kc, tid, u); offB[u] = x3_chunk_offset(b_kc, tid, u); }
        for (; kt + 2 < nk; ++kt) {
          AK_LDS3 unsigned char* cur = lds + (kt & 1) * BUF;
          AK_LDS3 unsigned char* nxt = lds + ((kt + 1) & 1) * BUF;
          const int k2 = kbeg + (kt + 2) * BK;
          // all LDS reads of this k-tile first: the stores into the other buffer cannot be proven not to alias
          bf16x8 fa[2][2][NSPLIT], fb[2][2][NSPLIT];
          auto read_frags = [&](int h) {
#pragma unroll
            for (int q = 0; q < NSPLIT; ++q) {
#pragma unroll
              for (int a = 0; a < 2; ++a) fa[h][a][q] = x3_frag(cur + q * X3_PLANE, a_kc, 64 * wr + 32 * a + l32, h, lane);
#pragma unroll
              for (int b = 0; b < 2; ++b)
                fb[h][b][q] = x3_frag(cur + (NSPLIT + q) * X3_PLANE, b_kc, 64 * wc + 32 * b + l32, h, lane);
            }
          };
          read_frags(0);
          read_frags(1);
          __builtin_amdgcn_sched_barrier(0);
          uint32_t pair[NSPLIT][2];
          x3_f32x2 rem;
#pragma unroll
          for (int m = 0; m < 48; ++m) {
            {   // matrix instruction m: (h, a, b) and the term, smallest terms first
              constexpr int PA[6] = {1, 0, 2, 0, 1, 0}, PB[6] = {1, 2, 0, 1, 0, 0};
              const int h = m / 24, ab = (m % 24) / 6, t = m % 6;
              constexpr int SM = CHUNKED ? 1 : 0;       // the cross products' accumulators exist in that variant only
              if (CHUNKED && t < 5)
                small[SM * (ab >> 1)][SM * (ab & 1)] =
                    mfma_bf16(fa[h][ab >> 1][PA[t]], fb[h][ab & 1][PB[t]], small[SM * (ab >> 1)][SM * (ab & 1)]);
              else
                acc[ab >> 1][ab & 1] = mfma_bf16(fa[h][ab >> 1][PA[t]], fb[h][ab & 1][PB[t]], acc[ab >> 1][ab & 1]);
            }
            {   // sixth m of the split: float4 u (0..3 of A, 4..7 of B), pair e, piece q
              const int u = m / 6, q = (m % 6) / 2, e = m % 2;
              const floatx4& v = u < 4 ? ra.v[u & 3] : rb.v[u & 3];
              if (q == 0) rem = x3_f32x2{v[2 * e], v[2 * e + 1]};
              else rem = x3_f32x2{v[2 * e], v[2 * e + 1]} - __builtin_convertvector(__builtin_bit_cast(x3_bf16x2, pair[0][e]), x3_f32x2)
                         - (q == 2 ? __builtin_convertvector(__builtin_bit_cast(x3_bf16x2, pair[1][e]), x3_f32x2) : x3_f32x2{0.f, 0.f});
              pair[q][e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rem, x3_bf16x2));
              if (m % 6 == 5) {
                AK_LDS3 unsigned char* dst = (u < 4 ? nxt + offA[u & 3] : nxt + NSPLIT * X3_PLANE + offB[u & 3]);
#pragma unroll
                for (int w = 0; w < NSPLIT; ++w) {
                  x3_u32x2 word;
                  word[0] = pair[w][0];
                  word[1] = pair[w][1];
                  *reinterpret_cast<AK_LDS3 x3_u32x2*>(dst + w * X3_PLANE) = word;
                }
                if (u < 4) ra.v[u & 3] = x3_fetch_one<INTERIOR>(A, p.lda, a_kc, i0, p.M, k2, kend, tid, u & 3);
                else rb.v[u & 3] = x3_fetch_one<INTERIOR>(B, p.ldb, b_kc, j0, p.N, k2, kend, tid, u & 3);
              }
            }
            __builtin_amdgcn_sched_barrier(0);
          }
          end_of_ktile(kt);
          __syncthreads();
        }
      }
      for (; kt < nk; ++kt) {
        AK_LDS3 unsigned char* cur = lds + (kt & 1) * BUF;
        AK_LDS3 unsigned char* nxt = lds + ((kt + 1) & 1) * BUF;
        if (kt + 1 < nk) stash(nxt);
        multiply(cur);
        end_of_ktile(kt);
        __syncthreads();
      }
    } else {
      __syncthreads();
      auto one_ktile = [&](int kt) {
        if (kt + 1 < nk) fetch(kt + 1);       // next k-tile's global loads fly during this one's MFMAs
        multiply(lds);
        __syncthreads();                      // everybody is done reading this k-tile
        if (kt + 1 < nk) stash(lds);
        __syncthreads();
      };
      if constexpr (CHUNKED) {
        // two nested loops: with one loop and a conditional flush the compiler evaluates the flush (a move and an
        // addition per accumulator register) at every k-tile and selects
        for (int kt0 = 0; kt0 < nk; kt0 += 8) {
          const int kt1 = kt0 + 8 < nk ? kt0 + 8 : nk;
          for (int kt = kt0; kt < kt1; ++kt) one_ktile(kt);
          end_of_ktile(7);
        }
      } else {
        for (int kt = 0; kt < nk; ++kt) one_ktile(kt);
      }
    }
  };
  if (interior) mainloop(std::true_type{});
  else mainloop(std::false_type{});
  (void)g; (void)panelA; (void)panelB;
  if constexpr (CHUNKED) {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          acc[a][b][r] = tot[a][b][r] + acc[a][b][r];
          if constexpr (NSPLIT >= 3) acc[a][b][r] += small[a][b][r];
        }
  }

  // the partial products of (i, j) and (j, i) are summed in different orders, so a mirrored result takes both
  // triangles of a diagonal tile from the lower one
  const bool mirror = (p.tile_mode == TILE_LOWER_MIRROR);
  const bool lower_only = (p.tile_mode == TILE_LOWER) || (mirror && ti == tj);
  if (p.beta != 0.f) {
    // all loads of C first: interleaved with the stores they would wait for one another (the compiler cannot tell
    // that the rows differ), one memory latency per element
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int gj = j0 + 64 * wc + 32 * b + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int gi = i0 + 64 * wr + 32 * a + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
          float c = 0.f;
          if (gj < p.N && gi < p.M && !(lower_only && gi < gj)) c = C[static_cast<int64_t>(gi) * p.ldc + gj];
          acc[a][b][r] = p.alpha * acc[a][b][r] + p.beta * c;
        }
      }
  } else {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] *= p.alpha;
  }
  float* __restrict__ C2 = p.C2 != nullptr ? p.C2 + static_cast<int64_t>(z) * p.sC2 : nullptr;
  float vmax = 0.f;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int gj = j0 + 64 * wc + 32 * b + l32;
      if (gj >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gi = i0 + 64 * wr + 32 * a + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (gi >= p.M) continue;
        if (lower_only && gi < gj) continue;
        const float v = acc[a][b][r];
        vmax = gemm_fold_absmax(vmax, v, gi == gj, p.absmax_identity);
        C[static_cast<int64_t>(gi) * p.ldc + gj] = v;
        if (mirror && gi != gj) C[static_cast<int64_t>(gj) * p.ldc + gi] = v;
        if (C2 != nullptr) {
          const float w = p.c2_scale * v + (gi == gj ? p.c2_diag : 0.f);
          C2[static_cast<int64_t>(gi) * p.ldc2 + gj] = w;
          if (mirror && gi != gj) C2[static_cast<int64_t>(gj) * p.ldc2 + gi] = w;
        }
      }
    }
  if (p.absmax_out != nullptr) gemm_store_absmax(p.absmax_out + static_cast<int64_t>(z) * p.absmax_stride, vmax, lane);
}

template <int NSPLIT, bool DB, int AKC = -1, int BKC = -1, bool CHUNKED = false>
static __global__ __launch_bounds__(256) void gemm_x3_kernel(GemmParams p) {
  __shared__ __attribute__((aligned(16))) unsigned char x3_smem[(DB ? 2 : 1) * 2 * NSPLIT * X3_PLANE];
  int ti = blockIdx.y, tj = blockIdx.x;
  if (p.tile_mode & TILE_LINEAR_GRID) {       // a launch of the lower tiles only: no work groups that exit at once
    p.tile_mode &= ~TILE_LINEAR_GRID;
    decode_lower_tile(blockIdx.x, ti, tj);
  }
  gemm_x3_tile<NSPLIT, DB, AKC, BKC, false, CHUNKED>(p, ti, tj, blockIdx.z, (AK_LDS3 unsigned char*)x3_smem);
}

// Grouped products: many independent C_i <- alpha_i * op(A_i) op(B_i) + beta_i * C_i of different sizes in one
// launch, so that products too small to fill the device share it and nothing waits on the host between them.
// `table` holds one row of GROUPED_ROW int64 per product: A, B, C, lda, ldb, ldc, M, N, K,
// transA | transB << 1 | symmetric << 2 (symmetric: M == N and the result is known to be symmetric, only the tiles
// on and below the diagonal are computed and mirrored), alpha and beta (float bits in the low and high word),
// first tile, then three optional addresses of float words: the largest magnitude in A, in B (from which the fp16-piece
// kernel takes its operand scales; required there) and where to fold the largest magnitude of the result (any split
// kernel), one spare.  Tiles are numbered row-major inside a product, products in table order (longest
// contraction first gives the best balance); work group w looks its product up by bisection on `first tile`.
constexpr int GROUPED_ROW = 16;

// Product and tile of work group w of a grouped launch; false for a tile the table overstates.
__device__ __forceinline__ int grouped_row_of(const int64_t* __restrict__ table, int count, int w) {
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[static_cast<int64_t>(mid) * GROUPED_ROW + 11] <= w) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

__device__ __forceinline__ bool grouped_lookup(const int64_t* __restrict__ table, int count, int w, GemmParams& p,
                                               int& ti, int& tj) {
  const int lo = grouped_row_of(table, count, w);
  const int64_t* __restrict__ r = table + static_cast<int64_t>(lo) * GROUPED_ROW;
  p.A = reinterpret_cast<const float*>(r[0]);
  p.B = reinterpret_cast<const float*>(r[1]);
  p.C = reinterpret_cast<float*>(r[2]);
  p.C_list = nullptr;
  p.lda = r[3]; p.ldb = r[4]; p.ldc = r[5];
  p.sA = p.sB = p.sC = 0;
  p.M = static_cast<int>(r[6]); p.N = static_cast<int>(r[7]); p.K = static_cast<int>(r[8]);
  p.transA = static_cast<int>(r[9] & 1); p.transB = static_cast<int>((r[9] >> 1) & 1);
  p.alpha = __builtin_bit_cast(float, static_cast<uint32_t>(r[10]));
  p.beta = __builtin_bit_cast(float, static_cast<uint32_t>(static_cast<uint64_t>(r[10]) >> 32));
  p.kmode = K_FULL;
  p.tile_mode = (r[9] & 4) ? TILE_LOWER_MIRROR : TILE_ALL;     // symmetric result: lower tiles only, mirrored
  p.active = nullptr; p.active_stride = 0;
  p.split = 0;
  p.chunked = 0;
  p.scaleA = p.scaleB = 1.f;
  p.absmax_out = reinterpret_cast<float*>(r[14]);
  const int local = w - static_cast<int>(r[11]);
  const int tn = (p.N + X3_BT - 1) / X3_BT;
  ti = local / tn;
  tj = local - ti * tn;
  return ti * X3_BT < p.M;
}

// The power of two that brings magnitudes up to `absmax` into (2^13, 2^14] (1 for zero, infinite or NaN input).
__device__ __forceinline__ float x3_half_scale(float absmax) {
  if (!(absmax > 0.f) || !(absmax < 3.0e38f)) return 1.f;
  int e;
  frexpf(absmax, &e);                  // absmax <= 2^e
  return ldexpf(1.f, 14 - e);
}

template <int NSPLIT, bool HALF = false, bool CHUNKED = false>
static __global__ __launch_bounds__(256, 2) void gemm_x3_grouped_kernel(const int64_t* __restrict__ table, int count) {
  __shared__ __attribute__((aligned(16))) unsigned char x3_smem[2 * NSPLIT * X3_PLANE];
  GemmParams p;
  int ti, tj;
  if (!grouped_lookup(table, count, blockIdx.x, p, ti, tj)) return;
  if constexpr (HALF) {
    // fp16 pieces: the operands' largest magnitudes (device words named by the table row) give the scales
    const int64_t* __restrict__ r = table + static_cast<int64_t>(grouped_row_of(table, count, blockIdx.x)) * GROUPED_ROW;
    p.scaleA = x3_half_scale(*reinterpret_cast<const float*>(r[12]));
    p.scaleB = x3_half_scale(*reinterpret_cast<const float*>(r[13]));
    p.alpha = p.alpha / (p.scaleA * p.scaleB);       // powers of two: exact
  }
  // two work groups per CU with the single-buffered loop serve the mix of long and short contractions of a
  // grouped launch better than one work group with the double-buffered loop (measured: 0.99 against 1.25 ms)
  gemm_x3_tile<NSPLIT, false, -1, -1, HALF, CHUNKED>(p, ti, tj, 0, (AK_LDS3 unsigned char*)x3_smem);
}

// The same with true fp32 products (v_mfma_f32_32x32x2_f32, one accumulation per k): 128 x 128 tiles as above.
static __global__ __launch_bounds__(256) void gemm_f32_grouped_kernel(const int64_t* __restrict__ table, int count) {
  __shared__ __attribute__((aligned(16))) float lds[2][2][GemmTile<128>::PANEL];
  GemmParams p;
  int ti, tj;
  if (!grouped_lookup(table, count, blockIdx.x, p, ti, tj)) return;
  gemm_f32_tile<2>(p, ti, tj, 0, lds);
}

// The split kernel takes operands whose 16-byte chunks never straddle the end of a row.
inline bool gemm_x3_ok(const GemmParams& p) {
  const int innerA = p.transA == 0 ? p.K : p.M, innerB = p.transB != 0 ? p.K : p.N;
  return p.lda % 4 == 0 && p.ldb % 4 == 0 && p.sA % 4 == 0 && p.sB % 4 == 0 && innerA % 4 == 0 && innerB % 4 == 0 &&
         (reinterpret_cast<uintptr_t>(p.A) & 15) == 0 && (reinterpret_cast<uintptr_t>(p.B) & 15) == 0;
}

}  // namespace ak
