// Products of symmetric fp32 matrices that are kept as three bf16 planes each (hi = x rounded to the nearest bf16,
// mid = x - hi rounded, lo = x - hi - mid, which is exact: hi + mid + lo == x), for iterations whose every matrix is
// the result of such a product (the coupled Newton iteration of the inverse roots): the split is paid once per
// element in the epilogue of the product that makes it, not once per tile that reads it, and the k-loop is the
// direct-to-LDS loop of the rank-k kernels (syrk_dtl_tile.hpp) with nothing for the vector ALU to do.
//
//   C = A B  with A, B, C symmetric n x n:  C[i][j] = sum_k A[k][i] B[k][j],
// so both operand panels are [32 rows k][columns] blocks of a row-major matrix, exactly what that loop loads.  The
// six piece products that matter (see gemm_x3.hpp) are formed from the six plane panels of a k-tile, which are loaded
// once, smallest terms first; the accumulators of 8 k-tiles (256 k) are added to a running total and start again
// from zero, which keeps the rounding error of a long sum near that of one rounding.  Tiles on and above the diagonal are computed and mirrored, a diagonal tile from its upper
// triangle: the result is exactly symmetric, which the next product, reading it as its own transpose, relies on.  The epilogue splits the result into its planes and can, in the same pass, write the planes of
// c2_scale * C + c2_diag * I and fold max |C - I| into a device word (a NaN is kept, as torch.max keeps it).
//
// Storage of one matrix: three planes of n_pad x n_pad bf16, n_pad a multiple of the 192-wide tile, zero outside
// the n x n corner: products of padded matrices stay zero there, and no load or store needs a bounds test.  A plane
// is stored by blocks of 32 columns, [n_pad / 32][n_pad rows][32 columns] (plane_index): the 16 rows x 64 bytes that
// one wave-wide load brings into the LDS are then one contiguous kilobyte, eight whole cache lines, instead of
// sixteen half lines a row apart.
//
// Second form, two fp16 planes (NP = 2): hi = s x rounded to the nearest fp16, lo = s x - hi rounded, with a power
// of two s per matrix that the caller picks so that s |x| stays below the fp16 maximum.  hi + lo holds 22 bits of
// s x and everything down to 2^-25 absolutely (the matrix instruction takes fp16 denormals as they are): for a matrix
// whose entries are bounded, e.g. a polynomial of a normalised symmetric matrix, that is the accuracy of an fp32
// product, whose accumulation rounds at 2^-24 of the sum anyway, for three piece products (hi hi, hi lo, lo hi)
// instead of six and two thirds of the operand bytes.  The accumulators hold s_A s_B C; the epilogue multiplies by
// `in_unscale` = 1 / (s_A s_B) and writes the planes of c_scale C.
#pragma once
#include "gemm_f32.hpp"
#include "syrk_dtl_tile.hpp"

namespace ak {

constexpr int kPlaneTile = 192;
constexpr int kPlaneLdsBytes = 4 * 6 * 6 * 16 * 64;      // four stages of six plane panels of six [16 rows][64 bytes] blocks
constexpr int kPlaneMaxDim = 16128;      // 32-bit byte offsets inside a plane set, virtual k-tile numbers below 2^15
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

struct PlaneGemm {
  const __bf16* A;          // plane set of batch entry z at A + z * set_elems (plane q: + q * plane_elems)
  const __bf16* B;
  __bf16* C;
  __bf16* C2;               // optional
  float* errword;           // optional, one word per batch entry
  const int* active;        // optional: entry z runs only if active[z] != 0
  int* overflow;            // optional, fp16 form: word z is set when a value of C or C2 does not fit the fp16 range
  int64_t sA, sB, sC, sC2;  // elements between the plane sets of consecutive batch entries
  int64_t plane_elems;      // n_pad * n_pad
  int n, n_pad, T;          // T = n_pad / kPlaneTile
  float c2_scale, c2_diag;
  // fp16 form only (powers of two): 1 / (scale of A's planes * scale of B's), scale of C's planes, scale of C2's
  float in_unscale, c_scale, c2_plane_scale;
};

// Element (i, j) of a plane stored by blocks of 32 columns.
__host__ __device__ __forceinline__ int64_t plane_index(int64_t i, int64_t j, int64_t n_pad) {
  return ((j >> 5) * n_pad + i) * 32 + (j & 31);
}

// The planes of x as 16-bit patterns.  NP = 3: bf16 hi, mid, lo (round to nearest each; the third remainder has at most
// 8 significant bits, so hi + mid + lo == x).  NP = 2: fp16 hi, lo of x, which the caller has scaled into range.
template <int NP>
__device__ __forceinline__ void plane_bits(float x, unsigned short (&o)[3]) {
  if constexpr (NP == 3) {
    const __bf16 hi = static_cast<__bf16>(x);
    const float r1 = x - static_cast<float>(hi);
    const __bf16 mid = static_cast<__bf16>(r1);
    const __bf16 lo = static_cast<__bf16>(r1 - static_cast<float>(mid));
    o[0] = __builtin_bit_cast(unsigned short, hi);
    o[1] = __builtin_bit_cast(unsigned short, mid);
    o[2] = __builtin_bit_cast(unsigned short, lo);
  } else {
    const _Float16 hi = static_cast<_Float16>(x);
    const _Float16 lo = static_cast<_Float16>(x - static_cast<float>(hi));
    o[0] = __builtin_bit_cast(unsigned short, hi);
    o[1] = __builtin_bit_cast(unsigned short, lo);
    o[2] = 0;
  }
}
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

// Epilogue of a tile: planes of C (and of C2 = c2_scale C + c2_diag I), the mirror image of an off-diagonal tile, the
// error word max |C - I|.  sum(a, b, r): the tile's sums in the accumulator layout of the 2 x 2 waves with 3 x 3 blocks each.
template <int NP, class Sum>
__device__ __forceinline__ void plane_epilogue(const PlaneGemm& p, int ti, int tj, int z, Sum sum) {
  constexpr int FR = 3, FC = 3, WC = 2;
  // (the empty statement keeps the address arithmetic below from being moved above the k-loop of the caller, where
  // every register is taken)
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = tid >> 6;
  const int wr = wave / WC, wc = wave % WC, g = lane >> 5, l32 = lane & 31;
  const int i0 = ti * kPlaneTile, j0 = tj * kPlaneTile;
  unsigned short* __restrict__ C = reinterpret_cast<unsigned short*>(p.C) + static_cast<int64_t>(z) * p.sC;
  unsigned short* __restrict__ C2 =
      p.C2 != nullptr ? reinterpret_cast<unsigned short*>(p.C2) + static_cast<int64_t>(z) * p.sC2 : nullptr;
  const bool off_diag = ti != tj;
  const float unscale = NP == 2 ? p.in_unscale : 1.f, cs = NP == 2 ? p.c_scale : 1.f, c2s = NP == 2 ? p.c2_plane_scale : 1.f;
  float vmax = 0.f;
  bool fits = true;
  // one 32 x 32 block of the wave; the block numbers are compile-time constants (a loop the compiler does not unroll
  // would index the accumulators with a variable, i.e. keep them in memory)
  auto block = [&](auto a_tag, auto b_tag) {
    constexpr int a = decltype(a_tag)::value, b = decltype(b_tag)::value;
    {
      const int gj = j0 + 32 * FC * wc + 32 * b + l32;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int gi = i0 + 32 * FR * wr + 32 * a + 8 * q + 4 * g;      // rows gi .. gi + 3
        u16x4 m1[NP], m2[NP];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = sum(a, b, 4 * q + e) * unscale;
          const bool inside = gi + e < p.n && gj < p.n, diagonal = gi + e == gj;
          if (inside && (off_diag || gi + e <= gj)) vmax = gemm_fold_absmax(vmax, v, diagonal, 1);
          unsigned short o[3];
          if constexpr (NP == 2) fits = fits && fabsf(v * cs) <= 65504.f;      // (false for a NaN too)
          plane_bits<NP>(v * cs, o);
          // a diagonal tile keeps its upper triangle and mirrors it element by element: the next product reads
          // this matrix as its own transpose, which it has to be exactly
          const bool keep = off_diag || gi + e <= gj;
          const int64_t at = plane_index(gi + e, gj, p.n_pad);
          const int64_t mirror = plane_index(gj, gi + e, p.n_pad);
#pragma unroll
          for (int s = 0; s < NP; ++s) {
            if (keep) C[s * p.plane_elems + at] = o[s];
            if (!off_diag && gi + e < gj) C[s * p.plane_elems + mirror] = o[s];
            m1[s][e] = o[s];
          }
          if (C2 != nullptr) {
            const float w = p.c2_scale * v + ((diagonal && inside) ? p.c2_diag : 0.f);
            if constexpr (NP == 2) fits = fits && fabsf(w * c2s) <= 65504.f;
            plane_bits<NP>(w * c2s, o);
#pragma unroll
            for (int s = 0; s < NP; ++s) {
              if (keep) C2[s * p.plane_elems + at] = o[s];
              if (!off_diag && gi + e < gj) C2[s * p.plane_elems + mirror] = o[s];
              m2[s][e] = o[s];
            }
          }
        }
        if (off_diag) {        // C[gj][gi .. gi + 3]: four consecutive elements of a row (gi is a multiple of 4)
          const int64_t at = plane_index(gj, gi, p.n_pad);
#pragma unroll
          for (int s = 0; s < NP; ++s) {
            *reinterpret_cast<u16x4*>(C + s * p.plane_elems + at) = m1[s];
            if (C2 != nullptr) *reinterpret_cast<u16x4*>(C2 + s * p.plane_elems + at) = m2[s];
          }
        }
      }
    }
  };
  using J0 = std::integral_constant<int, 0>;
  using J1 = std::integral_constant<int, 1>;
  using J2 = std::integral_constant<int, 2>;
  block(J0{}, J0{}); block(J0{}, J1{}); block(J0{}, J2{});
  block(J1{}, J0{}); block(J1{}, J1{}); block(J1{}, J2{});
  block(J2{}, J0{}); block(J2{}, J1{}); block(J2{}, J2{});
  if (p.errword != nullptr) gemm_store_absmax(p.errword + z, vmax, lane);
  if (NP == 2 && p.overflow != nullptr && !fits) atomicOr(p.overflow + z, 1);
}

// One 192 x 192 tile (ti <= tj) of batch entry z.  4 waves (2 x 2), 3 x 3 blocks of 32 x 32 per wave.
// A k-tile is 16 rows of all six planes (three of A's column block ti, three of B's column block tj): 36 KB of LDS per
// stage, four stages.  Per k-tile and wave: 6 pairs of planes x 9 matrix instructions, 9 wave-wide 16-byte loads (a
// load fills the 16 rows x 64 bytes of one 32-column block), one barrier.  The loads run two and a half k-tiles ahead
// (what they miss in the L2 takes microseconds to arrive); the barrier sits in the middle of a k-tile, so that the
// second half can already read the first fragments of the next one.
__device__ __forceinline__ void plane_tile(const PlaneGemm& p, int ti, int tj, int z) {
  constexpr int WR = 2, WC = 2, FR = 3, FC = 3, NCB = 6, BK = 16, S = 4;
  constexpr int BT = 32 * FR * WR;
  constexpr int BLOCK = BK * 64;                   // one 32-column block of one plane: [16 rows][64 bytes]
  constexpr int PANEL = NCB * BLOCK;               // one plane of one operand's 192 columns
  constexpr int STAGE = 6 * PANEL;                 // planes 0..2 of A's panel, then planes 0..2 of B's
  constexpr int LOADS = 6 * NCB / (WR * WC);       // wave-wide loads per wave and k-tile
  constexpr int CHUNK = 16;                        // k-tiles per partial sum (256 k)
  static_assert(BT == kPlaneTile && S * STAGE == kPlaneLdsBytes, "tile geometry");
  extern __shared__ __attribute__((aligned(1024))) unsigned char dtl_smem[];
  AK_LDS unsigned char* lds = (AK_LDS unsigned char*)dtl_smem;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
  if (p.active != nullptr && p.active[z] == 0) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / WC, wc = wave % WC;
  const int nk = p.n_pad / BK;
  const uint32_t plane_bytes = static_cast<uint32_t>(p.plane_elems) * 2u;

  u32x4 rsrc[2];
#pragma unroll
  for (int P = 0; P < 2; ++P) {
    const uint64_t ba = reinterpret_cast<uint64_t>(P == 0 ? p.A + static_cast<int64_t>(z) * p.sA
                                                          : p.B + static_cast<int64_t>(z) * p.sB);
    rsrc[P][0] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba));
    rsrc[P][1] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba >> 32) & 0xffffu);
    rsrc[P][2] = kDtlRange;
    rsrc[P][3] = 0x00020000u;
  }

  // The 36 blocks of a k-tile (operand P, plane q, column block cb) are dealt to the waves round-robin: wave w loads
  // blocks w, w + 4, ...; lane l brings row l / 4, 16-byte chunk l % 4 of the block's rows.
  // one block of one k-tile is 1 KB of consecutive bytes of the plane: block column (6 ti + cb), rows 16 kt ..
  const uint32_t lane_off = static_cast<uint32_t>(lane) * 16u;
  const uint32_t colblock_bytes = static_cast<uint32_t>(p.n_pad) * 64u;
  auto issue_load = [&](int kt, int stage, int l) {
    const uint32_t r = static_cast<uint32_t>(kt * BK) * 64u + lane_off;
    const int blk = wave + 4 * l;                  // 0 .. 35 = (P * 3 + q) * 6 + cb
    const int P = blk / 18, q = (blk / 6) % 3, cb = blk % 6;
    const uint32_t col = static_cast<uint32_t>((P == 0 ? ti : tj) * NCB + cb) * colblock_bytes;
    // (P differs between the waves of one instruction slot: both descriptors, one select)
    const u32x4 d = P == 0 ? rsrc[0] : rsrc[1];
    load_to_lds(d, lds0 + stage * STAGE + blk * BLOCK, kt < nk ? r + q * plane_bytes + col : 0u);
  };
  auto issue_loads = [&](int kt, int stage) {
#pragma unroll
    for (int l = 0; l < LOADS; ++l) issue_load(kt, stage, l);
  };

  floatx16 acc[FR][FC], tot[FR][FC];
#pragma unroll
  for (int a = 0; a < FR; ++a)
#pragma unroll
    for (int b = 0; b < FC; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) tot[a][b][r] = 0.f;

  const int g = lane >> 5, hl = (lane >> 4) & 1, j16 = lane & 15;
  const int frag_lane = (8 * g + (j16 >> 2)) * 64 + hl * 32 + (j16 & 3) * 8;
  AK_LDS const unsigned char* fragI = lds + frag_lane + wr * FR * BLOCK;
  AK_LDS const unsigned char* fragJ = lds + frag_lane + wc * FC * BLOCK + 3 * PANEL;

  auto tr = [](AK_LDS const unsigned char* q) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((AK_LDS short4v*)(q));
  };
  // A group = the FR (FC) fragments of one plane of A's (B's) panel for one k-tile.
  auto read_a = [&](bf16x8 (&f)[FR], int soff, int plane, int blk) {
    AK_LDS const unsigned char* q = fragI + soff + plane * PANEL + blk * BLOCK;
    f[blk] = pack_bf16x8(tr(q), tr(q + 256));
  };
  auto read_b = [&](bf16x8 (&f)[FC], int soff, int plane, int blk) {
    AK_LDS const unsigned char* q = fragJ + soff + plane * PANEL + blk * BLOCK;
    f[blk] = pack_bf16x8(tr(q), tr(q + 256));
  };
  bf16x8 fa[3][FR], fb[3][FC], fb0_next[FC];
  // The nine matrix instructions of one pair of planes, with the three fragment reads of a group that a later pair
  // needs spread between them (what: 0 none, 1 plane `plane` of A into fa[plane], 2 plane `plane` of B into fb[plane],
  // 3 plane 0 of B into fb0_next).
  // first_load >= 0: loads first_load .. first_load + 2 of k-tile load_kt go out one by one between the matrix
  // instructions (a wave alone on its SIMD cannot afford the issue time of nine in a row)
  auto pair_step = [&](const bf16x8 (&ca)[FR], const bf16x8 (&cb)[FC], auto what_tag, auto plane_tag, int soff,
                       int first_load = -1, int load_kt = 0) {
    constexpr int WHAT = decltype(what_tag)::value, PLANE = decltype(plane_tag)::value;
#pragma unroll
    for (int m = 0; m < FR * FC; ++m) {
      const int a = m / FC, b = m % FC;
      acc[a][b] = mfma_bf16(ca[a], cb[b], acc[a][b]);
      if (first_load >= 0 && m % 3 == 0) {
        __builtin_amdgcn_sched_barrier(0);
        issue_load(load_kt, load_kt & (S - 1), first_load + m / 3);
      }
      if (WHAT != 0 && m % 3 == 1) {
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (WHAT == 1) read_a(fa[PLANE], soff, PLANE, m / 3);
        if constexpr (WHAT == 2) read_b(fb[PLANE], soff, PLANE, m / 3);
        if constexpr (WHAT == 3) read_b(fb0_next, soff, 0, m / 3);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  // One k-tile: the six pairs in an order in which every step needs one new group only, smallest products first and
  // (hi, hi) last: (lo, hi), (mid, hi), (mid, mid), (hi, mid), (hi, lo), (hi, hi).  On entry fa[2] and b0 hold the
  // k-tile's first two groups; the last two steps fetch those of the next k-tile (plane 0 of B is in use until the
  // end, so it alternates between two register sets).
  auto ktile = [&](int kt, const bf16x8 (&b0)[FC], auto next_b0_tag) {
    constexpr int NEXT_B0 = decltype(next_b0_tag)::value;      // 2: into fb[0], 3: into fb0_next
    const int soff = (kt & (S - 1)) * STAGE, soff_next = ((kt + 1) & (S - 1)) * STAGE;
    pair_step(fa[2], b0, I1{}, I1{}, soff);
    pair_step(fa[1], b0, I2{}, I1{}, soff);
    pair_step(fa[1], fb[1], I1{}, I0{}, soff);
    // k-tile kt + 1 has landed for this wave (the loads of kt + 2 may still fly), then for all; and all waves are
    // done with k-tile kt - 1, whose stage the loads of k-tile kt + 3 fill
    wait_vmcnt<LOADS>();
    __syncthreads();
    pair_step(fa[0], fb[1], I2{}, I2{}, soff, 0, kt + 3);
    pair_step(fa[0], fb[2], I1{}, I2{}, soff_next, 3, kt + 3);
    if constexpr (NEXT_B0 == 3) pair_step(fa[0], b0, I3{}, I0{}, soff_next, 6, kt + 3);
    else pair_step(fa[0], b0, I2{}, I0{}, soff_next, 6, kt + 3);
  };

  issue_loads(0, 0);
  issue_loads(1, 1);
  issue_loads(2, 2);
  wait_vmcnt<2 * LOADS>();
  __syncthreads();
#pragma unroll
  for (int blk = 0; blk < 3; ++blk) { read_a(fa[2], 0, 2, blk); read_b(fb[0], 0, 0, blk); }
  // chunks of CHUNK k-tiles, each summed from zero and then added to the running total (two nested loops: with one
  // loop and a conditional reset the accumulators change register file at every k-tile)
  for (int kt0 = 0; kt0 < nk; kt0 += CHUNK) {
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
    const int kt1 = kt0 + CHUNK < nk ? kt0 + CHUNK : nk;      // (n_pad is a multiple of 192: an even number of k-tiles)
    for (int kt = kt0; kt < kt1; kt += 2) {
      ktile(kt, fb[0], I3{});
      ktile(kt + 1, fb0_next, I2{});
    }
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) tot[a][b][r] += acc[a][b][r];
  }
  wait_vmcnt<0>();                                             // the loads past the last k-tile, before the LDS is released

  plane_epilogue<3>(p, ti, tj, z, [&](int a, int b, int r) { return tot[a][b][r]; });
}

// The same tile on two fp16 planes per operand.  A k-tile is 16 rows of four plane panels (24 KB per stage, six
// stages: the loads run four and a half k-tiles ahead), three pairs of planes x 9 matrix instructions per wave:
// (lo, hi), (hi, hi), (hi, lo).  On entry fa[1] and fb[0] hold the k-tile's first two groups; the first two steps read
// the other two, the last one the first two groups of the next k-tile.
__device__ __forceinline__ void plane_tile_h2(const PlaneGemm& p, int ti, int tj, int z) {
  constexpr int WR = 2, WC = 2, FR = 3, FC = 3, NCB = 6, BK = 16, S = 6;
  constexpr int BT = 32 * FR * WR;
  constexpr int BLOCK = BK * 64;
  constexpr int PANEL = NCB * BLOCK;
  constexpr int STAGE = 4 * PANEL;                 // planes 0..1 of A's panel, then planes 0..1 of B's
  constexpr int LOADS = 4 * NCB / (WR * WC);
  constexpr int CHUNK = 16;
  static_assert(BT == kPlaneTile && S * STAGE == kPlaneLdsBytes, "tile geometry");
  extern __shared__ __attribute__((aligned(1024))) unsigned char dtl_smem[];
  AK_LDS unsigned char* lds = (AK_LDS unsigned char*)dtl_smem;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
  if (p.active != nullptr && p.active[z] == 0) return;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wr = wave / WC, wc = wave % WC;
  const int nk = p.n_pad / BK;
  const uint32_t plane_bytes = static_cast<uint32_t>(p.plane_elems) * 2u;

  u32x4 rsrc[2];
#pragma unroll
  for (int P = 0; P < 2; ++P) {
    const uint64_t ba = reinterpret_cast<uint64_t>(P == 0 ? p.A + static_cast<int64_t>(z) * p.sA
                                                          : p.B + static_cast<int64_t>(z) * p.sB);
    rsrc[P][0] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba));
    rsrc[P][1] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ba >> 32) & 0xffffu);
    rsrc[P][2] = kDtlRange;
    rsrc[P][3] = 0x00020000u;
  }
  // The 24 blocks of a k-tile (operand P, plane q, column block cb) are dealt to the waves round-robin.
  const uint32_t lane_off = static_cast<uint32_t>(lane) * 16u;
  const uint32_t colblock_bytes = static_cast<uint32_t>(p.n_pad) * 64u;
  auto issue_load = [&](int kt, int stage, int l) {
    const uint32_t r = static_cast<uint32_t>(kt * BK) * 64u + lane_off;
    const int blk = wave + 4 * l;                  // 0 .. 23 = (P * 2 + q) * 6 + cb
    const int P = blk / 12, q = (blk / 6) % 2, cb = blk % 6;
    const uint32_t col = static_cast<uint32_t>((P == 0 ? ti : tj) * NCB + cb) * colblock_bytes;
    const u32x4 d = P == 0 ? rsrc[0] : rsrc[1];
    load_to_lds(d, lds0 + stage * STAGE + blk * BLOCK, kt < nk ? r + q * plane_bytes + col : 0u);
  };
  auto issue_loads = [&](int kt, int stage) {
#pragma unroll
    for (int l = 0; l < LOADS; ++l) issue_load(kt, stage, l);
  };

  floatx16 acc[FR][FC], tot[FR][FC];
#pragma unroll
  for (int a = 0; a < FR; ++a)
#pragma unroll
    for (int b = 0; b < FC; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) tot[a][b][r] = 0.f;

  const int g = lane >> 5, hl = (lane >> 4) & 1, j16 = lane & 15;
  const int frag_lane = (8 * g + (j16 >> 2)) * 64 + hl * 32 + (j16 & 3) * 8;
  AK_LDS const unsigned char* fragI = lds + frag_lane + wr * FR * BLOCK;
  AK_LDS const unsigned char* fragJ = lds + frag_lane + wc * FC * BLOCK + 2 * PANEL;
  auto tr = [](AK_LDS const unsigned char* q) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((AK_LDS short4v*)(q));
  };
  bf16x8 fa[2][FR], fb[2][FC];                     // (fp16 patterns in 16-byte fragments)
  auto read_a = [&](int soff, int plane, int blk) {
    AK_LDS const unsigned char* q = fragI + soff + plane * PANEL + blk * BLOCK;
    fa[plane][blk] = pack_bf16x8(tr(q), tr(q + 256));
  };
  auto read_b = [&](int soff, int plane, int blk) {
    AK_LDS const unsigned char* q = fragJ + soff + plane * PANEL + blk * BLOCK;
    fb[plane][blk] = pack_bf16x8(tr(q), tr(q + 256));
  };
  using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
  // what: 1 plane 0 of A, 2 plane 1 of B (both of this k-tile), 3 plane 1 of A and plane 0 of B of the next k-tile
  // first_load >= 0: loads first_load .. first_load + 2 of k-tile load_kt go out one by one between the matrix
  // instructions (a wave alone on its SIMD cannot afford the issue time of six in a row)
  auto pair_step = [&](const bf16x8 (&ca)[FR], const bf16x8 (&cb)[FC], auto what_tag, int soff, int first_load, int load_kt,
                       int load_stage) {
    constexpr int WHAT = decltype(what_tag)::value;
#pragma unroll
    for (int m = 0; m < FR * FC; ++m) {
      const int a = m / FC, b = m % FC;
      acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, ca[a]), __builtin_bit_cast(f16x8, cb[b]),
                                                         acc[a][b], 0, 0, 0);
      if (first_load >= 0 && m % 3 == 0) {
        __builtin_amdgcn_sched_barrier(0);
        issue_load(load_kt, load_stage, first_load + m / 3);
      }
      if (m % 3 == 1) {
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (WHAT == 1) read_a(soff, 0, m / 3);
        if constexpr (WHAT == 2) read_b(soff, 1, m / 3);
        if constexpr (WHAT == 3) read_a(soff, 1, m / 3);
      }
      if (WHAT == 3 && m % 3 == 2) {
        __builtin_amdgcn_sched_barrier(0);
        read_b(soff, 0, m / 3);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;

#pragma unroll
  for (int t = 0; t < S - 1; ++t) issue_loads(t, t);
  wait_vmcnt<(S - 2) * LOADS>();
  __syncthreads();
#pragma unroll
  for (int blk = 0; blk < 3; ++blk) { read_a(0, 1, blk); read_b(0, 0, blk); }
  int stage = 0;                                   // kt % S
  for (int kt0 = 0; kt0 < nk; kt0 += CHUNK) {
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
    const int kt1 = kt0 + CHUNK < nk ? kt0 + CHUNK : nk;
    for (int kt = kt0; kt < kt1; ++kt) {
      const int next = stage + 1 == S ? 0 : stage + 1, fill = stage == 0 ? S - 1 : stage - 1;
      const int soff = stage * STAGE, soff_next = next * STAGE;
      pair_step(fa[1], fb[0], I1{}, soff, -1, 0, 0);
      // k-tile kt + 1 has landed for this wave, then for all; and all waves are done with k-tile kt - 1, whose stage
      // the loads of k-tile kt + S - 1 fill
      wait_vmcnt<(S - 3) * LOADS>();
      __syncthreads();
      pair_step(fa[0], fb[0], I2{}, soff, 0, kt + S - 1, fill);
      pair_step(fa[0], fb[1], I3{}, soff_next, 3, kt + S - 1, fill);
      stage = next;
    }
#pragma unroll
    for (int a = 0; a < FR; ++a)
#pragma unroll
      for (int b = 0; b < FC; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) tot[a][b][r] += acc[a][b][r];
  }
  wait_vmcnt<0>();
  plane_epilogue<2>(p, ti, tj, z, [&](int a, int b, int r) { return tot[a][b][r]; });
}

// Tile number -> (ti <= tj), in bands of 8 tile columns, row by row inside a band: the 32 work groups that share an
// L2 at any time then work on about 4 rows x 8 columns of tiles, i.e. read 4 + 8 column panels between them instead
// of the 2 + 16 of two rows of the triangle.  Band c (columns 8c .. 8c + w - 1, w = 8 but for the last) holds 8c rows of
// w tiles above its diagonal block and w, w - 1, .. 1 tiles in the block; bands before it hold 32 c^2 + 4 c tiles.
__device__ __forceinline__ void decode_banded_tile(int id, int T, int& ti, int& tj) {
  int c = static_cast<int>((__builtin_sqrtf(1.f + 32.f * static_cast<float>(id)) - 1.f) * (1.f / 16.f));
  while (32 * (c + 1) * (c + 1) + 4 * (c + 1) <= id) ++c;
  while (32 * c * c + 4 * c > id) --c;
  const int w = T - 8 * c < 8 ? T - 8 * c : 8;
  int local = id - (32 * c * c + 4 * c);
  if (local < 8 * c * w) {
    ti = local / w;
    tj = 8 * c + local - ti * w;
    return;
  }
  local -= 8 * c * w;
  int r = 0;
  while (local >= w - r) { local -= w - r; ++r; }
  ti = 8 * c + r;
  tj = ti + local;
}

// grid: tiles on and above the diagonal x batch, XCD-contiguous
template <int NP>
static __global__ __launch_bounds__(256) void plane_gemm_kernel(PlaneGemm p, int ntiles) {
  const uint32_t id = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int z = static_cast<int>(id / static_cast<uint32_t>(ntiles));
  int ti, tj;
  decode_banded_tile(static_cast<int>(id - static_cast<uint32_t>(z) * ntiles), p.T, ti, tj);
  if constexpr (NP == 3) plane_tile(p, ti, tj, z);
  else plane_tile_h2(p, ti, tj, z);
}

// planes: 3 (bf16) or 2 (fp16, with the scales of PlaneGemm)
inline int launch_plane_gemm(const PlaneGemm& p, int planes, int batch, hipStream_t stream) {
  constexpr int kLds = kPlaneLdsBytes;
  if (p.n_pad % kPlaneTile != 0 || p.n_pad > kPlaneMaxDim || p.T * kPlaneTile != p.n_pad || batch <= 0 ||
      (planes != 2 && planes != 3))
    return AK_ERR_ARG;
  static bool attr_set = false;     // idempotent; a race sets it twice at worst
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(plane_gemm_kernel<3>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLds) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(plane_gemm_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLds) != hipSuccess)
      return AK_ERR_LAUNCH;
    attr_set = true;
  }
  const int ntiles = p.T * (p.T + 1) / 2;
  if (planes == 3)
    hipLaunchKernelGGL(plane_gemm_kernel<3>, dim3(static_cast<unsigned>(ntiles) * batch), dim3(256), kLds, stream, p, ntiles);
  else
    hipLaunchKernelGGL(plane_gemm_kernel<2>, dim3(static_cast<unsigned>(ntiles) * batch), dim3(256), kLds, stream, p, ntiles);
  return check_launch();
}

}  // namespace ak
