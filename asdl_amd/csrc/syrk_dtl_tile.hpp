// Device side of the direct-to-LDS bf16 rank-k kernels: parameters, panel loads, the k-loop of one tile, the
// symmetric epilogue.  Shared by the factor kernels (syrk_dtl.hip) and the shifted-correlation form of the
// 3 x 3 convolution factors (conv_corr.hip).
//
// bf16 rank-k update C <- beta*C + alpha * U^T U whose panels travel global memory -> LDS without
// passing through registers (buffer_load_dwordx4 ... lds), for two kinds of U:
//   plain : U = X, a row-major [M, d] matrix (the contraction index is the strided one);
//   gather: U = the unfolded input of a convolution, never materialised.  x is [N, H, W, C] (channels
//           last); row (n,oy,ox) of U holds, for every tap (ky,kx), the C channels of input pixel
//           (oy*sh - ph + ky, ox*sw - pw + kx), zeros outside the image.  The kernel works in the
//           column order (c/G, ky, kx, c%G) for a group size G (a multiple of 8 dividing C): 8 consecutive
//           columns are 16 contiguous bytes of x.  The epilogue applies the permutation to the (c,ky,kx)
//           order of the dense factor, which stays inside blocks of G*kh*kw columns.  A column block of a
//           panel is 32 columns wide, so any G that is a multiple of 32 gives the loads the same 64 contiguous
//           bytes per row; the smaller G, the fewer cache lines the permuted 4-byte writes of a tile row are
//           spread over (G = 32: 18 lines, two thirds of each filled by one tile; measured 3-11 % faster than
//           G = 128).  G = 8 for the largest factors, whose direct epilogue writes 85 MB.
//
// One work group owns one BT x BT tile of the upper triangle and, with split-K, a slice of the M rows.
// A k-tile is 32 rows.  Per k-tile and panel the LDS holds BT/32 column blocks, each [32 rows][32 cols]
// bf16 with 64-byte rows: one wave-wide 16-byte load fills 16 rows of a block (lane l -> row l/4,
// 16-byte chunk l%4), so every lane keeps the same row for all its loads of a k-tile and the 64 bytes per
// row stay contiguous in global memory.  ds_read_b64_tr_b16 then finds, for the 32 lanes it serves per
// pass, 4 rows x 64 bytes = 256 consecutive bytes: no bank conflicts and no padding.
// The loads run STAGES-1 k-tiles ahead of the MFMAs; completion is tracked with s_waitcnt vmcnt, the
// hand-over between waves with one barrier per k-tile.  Rows and columns outside the matrix (or taps
// outside the image) are given a byte offset beyond the buffer range, for which the hardware returns
// zeros, so the main loop has no masks and no branches.
#pragma once
#include <type_traits>
#include "common.hpp"

namespace ak {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define AK_LDS __attribute__((address_space(3)))

constexpr int kDtlBK = 32;              // rows per k-tile
constexpr int kDtlStages = 4;          // >= 3: the loads run two k-tiles ahead of the one being read
constexpr uint32_t kDtlRange = 0xFFFFFF00u;   // num_records of the descriptor; larger offsets read as zero
constexpr uint32_t kDtlOob = 0xFFFFFFFFu;

struct DtlParams {
  const void* X;
  float* C;
  float* ws;
  int64_t M, d, ldc, rows_per_split;
  uint32_t row_bytes;      // plain: bytes between rows of X
  int T, nsplit;
  float alpha, beta;
  // gather geometry
  int Cin, H, W, kw, KK, sh, sw, ph, pw, Ho, Wo;
  int G;                          // channels per column group
  uint32_t mWo, mHo, mKw, mBlk, mG, mKK;   // magic multipliers: Wo, Ho, kw, G*KK, G, KK
};

// 16 bytes per lane, global -> LDS at m0 + 16*lane.  The compiler does not see the LDS write: callers
// order it against LDS reads with s_waitcnt vmcnt + a barrier.
__device__ __forceinline__ void load_to_lds(u32x4 rsrc, uint32_t lds_addr, uint32_t voff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :: "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  // gfx9 encoding: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14; expcnt/lgkmcnt left at "no wait"
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// Working column v = blk*(G*KK) + tap*G + cg stands for channel c = G*blk + cg and tap (ky,kx).
__device__ __forceinline__ void decode_column(uint32_t v, const DtlParams& p, uint32_t& c, uint32_t& tap) {
  const uint32_t blk = fastdiv(v, p.mBlk, p.G * p.KK);
  const uint32_t rem = v - blk * p.G * p.KK;
  tap = fastdiv(rem, p.mG, p.G);
  c = blk * p.G + rem - tap * p.G;
}

template <bool GATHER>
__device__ __forceinline__ int64_t out_index(int64_t v, const DtlParams& p) {
  if constexpr (!GATHER) return v;
  uint32_t c, tap;
  decode_column(static_cast<uint32_t>(v), p, c, tap);
  return static_cast<int64_t>(c * p.KK + tap);
}

// Writes one wave's accumulators: C[oi][oj] = beta*C + alpha*acc and the mirror off the diagonal tile.
template <int FR, int FC, bool GATHER>
__device__ __forceinline__ void dtl_epilogue(floatx16 (&acc)[FR][FC], const DtlParams& p, int64_t gi0, int64_t gj0,
                                             bool diag_tile, int lane) {
  if constexpr (!GATHER) {
    syrk_epilogue<FR, FC>(acc, p.C, p.ldc, p.d, gi0, gj0, diag_tile, p.alpha, p.beta, lane);
  } else {
    const int g = lane >> 5, l32 = lane & 31;
    // First acc <- alpha * acc + beta * C, then the stores, so that no read of C waits behind a store to C.  The
    // reads go through a buffer descriptor of C (see syrk_epilogue): the four rows of an accumulator float4 are
    // consecutive channels of one tap, KK result rows apart, so their row offsets are scalars; rows and columns
    // beyond d get an out-of-range offset and read as zero.
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] *= p.alpha;
    if (p.beta != 0.f) {
      // (results of 4 GiB and more are refused on the host: (d + 256) * d < 2^32 / 4 is required of gathered factors)
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
          p.C, 0, static_cast<int>(((p.d - 1) * p.ldc + p.d) * 4), 0x00020000);
      const uint32_t ldc4 = static_cast<uint32_t>(p.ldc) * 4u, row_step = static_cast<uint32_t>(p.KK) * ldc4;
      uint32_t row_off[FR][4];
#pragma unroll
      for (int a = 0; a < FR; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t gi = gi0 + 32 * a + 8 * q + 4 * g;
          row_off[a][q] = gi < p.d ? static_cast<uint32_t>(out_index<true>(gi, p)) * ldc4 : kDtlOob;
        }
#pragma unroll
      for (int b = 0; b < FC; ++b) {
        const int64_t gj = gj0 + 32 * b + l32;
        const uint32_t col_off = gj < p.d ? static_cast<uint32_t>(out_index<true>(gj, p)) * 4u : kDtlOob;
#pragma unroll
        for (int a = 0; a < FR; ++a)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const bool ok = row_off[a][q] != kDtlOob && col_off != kDtlOob;
            const uint32_t voff = ok ? row_off[a][q] + col_off : kDtlOob;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float c = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, e * row_step, 0));
              acc[a][b][4 * q + e] += p.beta * c;
            }
          }
      }
    }
#pragma unroll
    for (int b = 0; b < FC; ++b) {
      const int64_t gj = gj0 + 32 * b + l32;
      if (gj >= p.d) continue;
      const int64_t oj = out_index<true>(gj, p);
#pragma unroll
      for (int a = 0; a < FR; ++a) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t gi = gi0 + 32 * a + 8 * q + 4 * g;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (gi + e >= p.d) continue;
            const int64_t oi = out_index<true>(gi + e, p);
            const float v = acc[a][b][4 * q + e];
            p.C[oi * p.ldc + oj] = v;
            if (!diag_tile) p.C[oj * p.ldc + oi] = v;
          }
        }
      }
    }
  }
}

template <int WR, int WC, int FR, int FC, bool GATHER>
struct DtlCfg {
  static constexpr int NW = WR * WC;
  static constexpr int BT = 32 * FR * WR;
  static constexpr int NCB = BT / 32;                         // column blocks per panel
  static constexpr int BLOCK_BYTES = kDtlBK * 64;             // one column block of one k-tile
  static constexpr int PANEL_BYTES = NCB * BLOCK_BYTES;
  static constexpr int STAGE_BYTES = 2 * PANEL_BYTES;
  static constexpr int LDS_BYTES = kDtlStages * STAGE_BYTES;
  static constexpr int IPW = NCB * (kDtlBK / 16) / NW;        // wave-wide loads per wave, panel and k-tile
  static_assert(32 * FC * WC == BT, "square work-group tile");
  static_assert(NCB * (kDtlBK / 16) % NW == 0 && IPW >= 1, "loads must split evenly over the waves");
};

// Work groups go to the 8 XCDs round-robin by their linear index, and each XCD has its own L2.  Renumbering them so
// that one XCD gets a contiguous range of work items lets the tiles of one split share the rows they read through
// one L2 instead of fetching them once per XCD.
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t wgid, uint32_t nwg) {
  const uint32_t xcd = wgid & 7, local = wgid >> 3, q = nwg >> 3, rem = nwg & 7;
  return xcd * q + (xcd < rem ? xcd : rem) + local;
}

// Rows [k_begin, k_begin + rows) of the operand into tile (ti, tj) of one factor.  partial == nullptr: the result is
// the factor's tile (alpha, beta, mirror image); otherwise the accumulators go to `partial` in accumulator order,
// [(a, b, q)][thread] float4, for a reduction pass.  raw != nullptr: the bare tile goes to a row-major matrix.
template <int WR, int WC, int FR, int FC, bool GATHER>
__device__ __forceinline__ void dtl_tile(const DtlParams& p, int ti, int tj, int64_t k_begin, int rows,
                                         floatx4* __restrict__ partial, float* __restrict__ raw = nullptr,
                                         int64_t raw_ld = 0) {
  using Cfg = DtlCfg<WR, WC, FR, FC, GATHER>;
  constexpr int NW = Cfg::NW, BT = Cfg::BT, NCB = Cfg::NCB, IPW = Cfg::IPW, BK = kDtlBK, S = kDtlStages;
  extern __shared__ __attribute__((aligned(1024))) unsigned char dtl_smem[];
  AK_LDS unsigned char* lds = (AK_LDS unsigned char*)dtl_smem;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / WC, wc = wave % WC;
  const bool diag = (ti == tj);
  const int64_t i0 = static_cast<int64_t>(ti) * BT, j0 = static_cast<int64_t>(tj) * BT;
  const int nk = (rows + BK - 1) / BK;

  // buffer descriptor: plain mode is based at this split's first row, gather mode at the tensor
  const unsigned char* base = static_cast<const unsigned char*>(p.X);
  if constexpr (!GATHER) base += k_begin * static_cast<int64_t>(p.row_bytes);
  const uint64_t ba = reinterpret_cast<uint64_t>(base);
  u32x4 rsrc;
  rsrc[0] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba));
  rsrc[1] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba >> 32) & 0xffffu);
  rsrc[2] = kDtlRange;
  rsrc[3] = 0x00020000u;

  // this lane's part in the panel loads: one row of the k-tile, IPW 16-byte chunks per panel
  const int half = wave & 1;                       // rows 16*half .. 16*half+15 of the k-tile
  const int row_in_tile = 16 * half + (lane >> 2);
  const int cb0 = (wave >> 1) * IPW;               // first column block this wave loads
  uint32_t coloff[2][IPW];                         // byte offset of the chunk inside a row (kDtlOob: no such column)
  int tapy[2][IPW], tapx[2][IPW];
#pragma unroll
  for (int P = 0; P < 2; ++P) {
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
      const int64_t v = (P == 0 ? i0 : j0) + 32 * (cb0 + i) + 8 * (lane & 3);
      tapy[P][i] = tapx[P][i] = 0;
      if (v >= p.d) {
        coloff[P][i] = kDtlOob;
      } else if constexpr (!GATHER) {
        coloff[P][i] = static_cast<uint32_t>(v) * 2u;
      } else {
        uint32_t c, tap;
        decode_column(static_cast<uint32_t>(v), p, c, tap);
        const uint32_t ky = fastdiv(tap, p.mKw, p.kw), kx = tap - ky * p.kw;
        tapy[P][i] = ky;
        tapx[P][i] = kx;
        coloff[P][i] = ((ky * p.W + kx) * p.Cin + c) * 2u;
      }
    }
  }
  const uint32_t lds_lane_blk = lds0 + cb0 * Cfg::BLOCK_BYTES + half * 1024;   // + stage + panel + i*BLOCK_BYTES

  // Row part of the addresses of one k-tile (shared by all loads of the lane), then one load per call.
  struct RowState { uint32_t rowoff; int iy0, ix0; bool ok; uint32_t sbase; };
  auto prepare = [&](int kt, int stage) {
    RowState st;
    const int r = kt * BK + row_in_tile;           // row of this split
    st.ok = r < rows;
    st.iy0 = st.ix0 = 0;
    if constexpr (!GATHER) {
      st.rowoff = static_cast<uint32_t>(r) * p.row_bytes;
    } else {
      const uint32_t pos = static_cast<uint32_t>(k_begin) + r;
      const uint32_t q1 = fastdiv(pos, p.mWo, p.Wo);
      const uint32_t ox = pos - q1 * p.Wo;
      const uint32_t n = fastdiv(q1, p.mHo, p.Ho);
      const uint32_t oy = q1 - n * p.Ho;
      st.iy0 = static_cast<int>(oy) * p.sh - p.ph;
      st.ix0 = static_cast<int>(ox) * p.sw - p.pw;
      st.rowoff = static_cast<uint32_t>((static_cast<int>(n * p.H) + st.iy0) * p.W + st.ix0) *
                  static_cast<uint32_t>(p.Cin * 2);
    }
    st.sbase = lds_lane_blk + stage * Cfg::STAGE_BYTES;
    return st;
  };
  auto load_one = [&](const RowState& st, int P, int i) {
    bool ok = st.ok && coloff[P][i] != kDtlOob;
    if constexpr (GATHER)
      ok = ok && static_cast<unsigned>(st.iy0 + tapy[P][i]) < static_cast<unsigned>(p.H) &&
           static_cast<unsigned>(st.ix0 + tapx[P][i]) < static_cast<unsigned>(p.W);
    const uint32_t voff = ok ? st.rowoff + coloff[P][i] : kDtlOob;
    load_to_lds(rsrc, st.sbase + P * Cfg::PANEL_BYTES + i * Cfg::BLOCK_BYTES, voff);
  };

  floatx16 acc[FR][FC];
#pragma unroll
  for (int a = 0; a < FR; ++a)
#pragma unroll
    for (int b = 0; b < FC; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  // fragment addressing: lane (g, hl, j) reads row 8g + j/4 (+4 for the second half of the fragment),
  // bytes 32*hl + 8*(j%4) of its 64-byte row
  const int g = lane >> 5, hl = (lane >> 4) & 1, j16 = lane & 15;
  const int frag_lane = (8 * g + (j16 >> 2)) * 64 + hl * 32 + (j16 & 3) * 8;
  AK_LDS const unsigned char* fragI = lds + frag_lane + wr * FR * Cfg::BLOCK_BYTES;
  AK_LDS const unsigned char* fragJ = lds + frag_lane + wc * FC * Cfg::BLOCK_BYTES + (diag ? 0 : Cfg::PANEL_BYTES);

  auto tr = [](AK_LDS const unsigned char* q) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((AK_LDS short4v*)(q));
  };
  // fragment u of a half k-tile in the order the MFMAs want them: a0, b0 .. b(FC-1), a1 .. a(FR-1)
  auto read_unit = [&](bf16x8 (&fa)[FR], bf16x8 (&fb)[FC], int soff, int kk, int u) {
    if (u == 0 || u > FC) {
      const int a = u == 0 ? 0 : u - FC;
      AK_LDS const unsigned char* q = fragI + soff + a * Cfg::BLOCK_BYTES + kk * 64;
      fa[a] = pack_bf16x8(tr(q), tr(q + 256));
    } else {
      const int b = u - 1;
      AK_LDS const unsigned char* q = fragJ + soff + b * Cfg::BLOCK_BYTES + kk * 64;
      fb[b] = pack_bf16x8(tr(q), tr(q + 256));
    }
  };

  // One half k-tile (16 rows): FR*FC MFMAs on the fragments (ca, cb), with the LDS reads of the next half's
  // fragments (na, nb) and, if NLOAD > 0, the panel loads of a k-tile further ahead spread between them so
  // that the matrix pipe never waits for their issue.
  auto half_step = [&](auto nload_tag, const bf16x8 (&ca)[FR], const bf16x8 (&cb)[FC], bf16x8 (&na)[FR],
                       bf16x8 (&nb)[FC], int soff_next, int kk_next, const RowState& st) {
    constexpr int NLOAD = decltype(nload_tag)::value;
    constexpr int NM = FR * FC, NS = NLOAD + FR + FC;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      const int a = m / FC, b = m % FC;
      acc[a][b] = mfma_bf16(ca[a], cb[b], acc[a][b]);
#pragma unroll
      for (int sidx = (m * NS) / NM; sidx < ((m + 1) * NS) / NM; ++sidx) {
        __builtin_amdgcn_sched_barrier(0);
        if (sidx < NLOAD) load_one(st, sidx / IPW, sidx % IPW);
        else read_unit(na, nb, soff_next, kk_next, sidx - NLOAD);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  auto mainloop = [&](auto diag_tag) {
    constexpr bool DIAG = decltype(diag_tag)::value;
    constexpr int LPT = IPW * (DIAG ? 1 : 2);      // loads per wave and k-tile
#pragma unroll
    for (int t = 0; t < S - 1; ++t) {              // tiles beyond nk load zeros: the counts stay uniform
      const RowState st = prepare(t, t);
#pragma unroll
      for (int l = 0; l < LPT; ++l) load_one(st, l / IPW, l % IPW);
    }
    wait_vmcnt<(S - 2) * LPT>();                   // this wave's loads of k-tile 0 have landed
    __syncthreads();                               // ... and everybody's
    bf16x8 fa0[FR], fb0[FC], fa1[FR], fb1[FC];
#pragma unroll
    for (int u = 0; u < FR + FC; ++u) read_unit(fa0, fb0, 0, 0, u);
    int rd = 0, wrs = S - 1;
    const RowState none{};
    for (int kt = 0; kt < nk; ++kt) {
      // first half: MFMAs on rows 0..15 of k-tile kt while rows 16..31 come out of the LDS
      half_step(std::integral_constant<int, 0>{}, fa0, fb0, fa1, fb1, rd * Cfg::STAGE_BYTES, 16, none);
      wait_vmcnt<(S - 3) * LPT>();                 // own loads of k-tile kt+1 have landed
      __syncthreads();                             // everybody's have; nobody reads k-tile kt-1 any more
      // second half: MFMAs on rows 16..31 while k-tile kt+S-1 is requested into the stage k-tile kt-1
      // occupied and rows 0..15 of k-tile kt+1 come out of the LDS
      const RowState st = prepare(kt + S - 1, wrs);
      rd = (rd + 1 == S) ? 0 : rd + 1;
      wrs = (wrs + 1 == S) ? 0 : wrs + 1;
      half_step(std::integral_constant<int, LPT>{}, fa1, fb1, fa0, fb0, rd * Cfg::STAGE_BYTES, 0, st);
    }
    wait_vmcnt<0>();                               // drain the zero-fill loads before the LDS is released
  };
  if (diag) mainloop(std::true_type{});
  else mainloop(std::false_type{});

  const int64_t gi0 = i0 + 32 * FR * wr, gj0 = j0 + 32 * FC * wc;
  if (raw != nullptr) {
    // the tile as it is, row-major with leading dimension raw_ld at `raw` (no scaling, no mirror image, no bounds)
    const int g = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          raw[(32 * FR * wr + 32 * a + 8 * (r >> 2) + 4 * g + (r & 3)) * raw_ld + 32 * FC * wc + 32 * b + l32] = acc[a][b][r];
  } else if (partial == nullptr) {
    dtl_epilogue<FR, FC, GATHER>(acc, p, gi0, gj0, diag, lane);
  } else {
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          floatx4 w = {acc[a][b][4 * q], acc[a][b][4 * q + 1], acc[a][b][4 * q + 2], acc[a][b][4 * q + 3]};
          partial[((a * FC + b) * 4 + q) * (NW * 64) + tid] = w;
        }
  }
}

}  // namespace ak
