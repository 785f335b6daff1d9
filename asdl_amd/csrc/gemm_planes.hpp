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
// Storage of one matrix: three planes of [n_pad][n_pad] bf16, n_pad a multiple of the 192-wide tile, zero outside
// the n x n corner: products of padded matrices stay zero there, and no load or store needs a bounds test.
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
  int64_t sA, sB, sC, sC2;  // elements between the plane sets of consecutive batch entries
  int64_t plane_elems;      // n_pad * n_pad
  int n, n_pad, T;          // T = n_pad / kPlaneTile
  float c2_scale, c2_diag;
};

// The three planes of x (round to nearest each; the third remainder has at most 8 significant bits).
__device__ __forceinline__ void plane_split(float x, __bf16& hi, __bf16& mid, __bf16& lo) {
  hi = static_cast<__bf16>(x);
  const float r1 = x - static_cast<float>(hi);
  mid = static_cast<__bf16>(r1);
  lo = static_cast<__bf16>(r1 - static_cast<float>(mid));
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
  const int i0 = ti * BT, j0 = tj * BT;
  const int nk = p.n_pad / BK;
  const uint32_t row_bytes = static_cast<uint32_t>(p.n_pad) * 2u;
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
  const uint32_t lane_off = static_cast<uint32_t>(lane >> 2) * row_bytes + static_cast<uint32_t>(lane & 3) * 16u;
  auto issue_loads = [&](int kt, int stage) {
    const uint32_t r = static_cast<uint32_t>(kt * BK) * row_bytes + lane_off;
#pragma unroll
    for (int l = 0; l < LOADS; ++l) {
      const int blk = wave + 4 * l;                // 0 .. 35 = (P * 3 + q) * 6 + cb
      const int P = blk / 18, q = (blk / 6) % 3, cb = blk % 6;
      const uint32_t col = static_cast<uint32_t>((P == 0 ? i0 : j0) + 32 * cb) * 2u;
      // (P differs between the waves of one instruction slot: both descriptors, one select)
      const u32x4 d = P == 0 ? rsrc[0] : rsrc[1];
      load_to_lds(d, lds0 + stage * STAGE + blk * BLOCK, kt < nk ? r + q * plane_bytes + col : 0u);
    }
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
  auto pair_step = [&](const bf16x8 (&ca)[FR], const bf16x8 (&cb)[FC], auto what_tag, auto plane_tag, int soff) {
    constexpr int WHAT = decltype(what_tag)::value, PLANE = decltype(plane_tag)::value;
#pragma unroll
    for (int m = 0; m < FR * FC; ++m) {
      const int a = m / FC, b = m % FC;
      acc[a][b] = mfma_bf16(ca[a], cb[b], acc[a][b]);
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
    issue_loads(kt + 3, (kt + 3) & (S - 1));
    pair_step(fa[0], fb[1], I2{}, I2{}, soff);
    pair_step(fa[0], fb[2], I1{}, I2{}, soff_next);
    if constexpr (NEXT_B0 == 3) pair_step(fa[0], b0, I3{}, I0{}, soff_next);
    else pair_step(fa[0], b0, I2{}, I0{}, soff_next);
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

  // epilogue: planes of C (and of C2), the mirror image of an off-diagonal tile, the error word
  const int l32 = lane & 31;
  __bf16* __restrict__ C = p.C + static_cast<int64_t>(z) * p.sC;
  __bf16* __restrict__ C2 = p.C2 != nullptr ? p.C2 + static_cast<int64_t>(z) * p.sC2 : nullptr;
  const bool off_diag = ti != tj;
  float vmax = 0.f;
#pragma unroll
  for (int a = 0; a < FR; ++a)
#pragma unroll
    for (int b = 0; b < FC; ++b) {
      const int gj = j0 + 32 * FC * wc + 32 * b + l32;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int gi = i0 + 32 * FR * wr + 32 * a + 8 * q + 4 * g;      // rows gi .. gi + 3
        bf16x4 m1[3], m2[3];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = tot[a][b][4 * q + e];
          const bool inside = gi + e < p.n && gj < p.n, diagonal = gi + e == gj;
          if (inside && (off_diag || gi + e <= gj)) vmax = gemm_fold_absmax(vmax, v, diagonal, 1);
          __bf16 h, m, l;
          plane_split(v, h, m, l);
          // a diagonal tile keeps its upper triangle and mirrors it element by element: the next product reads
          // this matrix as its own transpose, which it has to be exactly
          const bool keep = off_diag || gi + e <= gj;
          const int64_t at = static_cast<int64_t>(gi + e) * p.n_pad + gj;
          const int64_t mirror = static_cast<int64_t>(gj) * p.n_pad + gi + e;
          if (keep) { C[at] = h; C[p.plane_elems + at] = m; C[2 * p.plane_elems + at] = l; }
          if (!off_diag && gi + e < gj) { C[mirror] = h; C[p.plane_elems + mirror] = m; C[2 * p.plane_elems + mirror] = l; }
          m1[0][e] = h; m1[1][e] = m; m1[2][e] = l;
          if (C2 != nullptr) {
            const float w = p.c2_scale * v + ((diagonal && inside) ? p.c2_diag : 0.f);
            plane_split(w, h, m, l);
            if (keep) { C2[at] = h; C2[p.plane_elems + at] = m; C2[2 * p.plane_elems + at] = l; }
            if (!off_diag && gi + e < gj) { C2[mirror] = h; C2[p.plane_elems + mirror] = m; C2[2 * p.plane_elems + mirror] = l; }
            m2[0][e] = h; m2[1][e] = m; m2[2][e] = l;
          }
        }
        if (off_diag) {        // C[gj][gi .. gi + 3]: four consecutive elements of a row
          const int64_t at = static_cast<int64_t>(gj) * p.n_pad + gi;
#pragma unroll
          for (int s = 0; s < 3; ++s) {
            *reinterpret_cast<bf16x4*>(C + s * p.plane_elems + at) = m1[s];
            if (C2 != nullptr) *reinterpret_cast<bf16x4*>(C2 + s * p.plane_elems + at) = m2[s];
          }
        }
      }
    }
  if (p.errword != nullptr) gemm_store_absmax(p.errword + z, vmax, lane);
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
static __global__ __launch_bounds__(256) void plane_gemm_kernel(PlaneGemm p, int ntiles) {
  const uint32_t id = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int z = static_cast<int>(id / static_cast<uint32_t>(ntiles));
  int ti, tj;
  decode_banded_tile(static_cast<int>(id - static_cast<uint32_t>(z) * ntiles), p.T, ti, tj);
  plane_tile(p, ti, tj, z);
}

inline int launch_plane_gemm(const PlaneGemm& p, int batch, hipStream_t stream) {
  constexpr int kLds = kPlaneLdsBytes;
  if (p.n_pad % kPlaneTile != 0 || p.n_pad > kPlaneMaxDim || p.T * kPlaneTile != p.n_pad || batch <= 0) return AK_ERR_ARG;
  static bool attr_set = false;     // idempotent; a race sets it twice at worst
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(plane_gemm_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kLds) != hipSuccess)
      return AK_ERR_LAUNCH;
    attr_set = true;
  }
  const int ntiles = p.T * (p.T + 1) / 2;
  hipLaunchKernelGGL(plane_gemm_kernel, dim3(static_cast<unsigned>(ntiles) * batch), dim3(256), kLds, stream, p,
                     ntiles);
  return check_launch();
}

}  // namespace ak
