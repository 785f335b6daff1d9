// Input factor A = U^T U of a 3 x 3 convolution with stride 1 and padding 1 on a channels-last bf16 input, from
// shifted correlations of the input instead of the unfolded matrix U (asdl/operations/conv.py:80-88 forms
// U U^T of the unfolded input; the result here is that matrix, summed in a different order).
//
// Block (t, t') of A, t = (ky, kx), is  sum over output positions o of  x[o + t - 1]^T x[o + t' - 1]  (x zero outside
// the image).  With p = o + t - 1 and D = t' - t that is  sum_p x[p]^T x[p + D]  over the pixels p whose output
// position lies inside the image.  The sum over ALL pixels, R_D, depends on the shift D only: 25 shifts, of which 13
// are distinct up to transposition (R_-D = R_D^T), replace the 45 distinct blocks, and each R_D is a product of the
// [N H W, C] pixel matrix with a row-shifted view of itself.  What R_D counts too often are the pixels p whose
// output position o = p - t + 1 falls outside the image: image row H-1 for ky = 0, row 0 for ky = 2, and the same
// for columns.  A pixel of such a row has p + D inside the image only if D_y = 0, so the corrections are
//   D_y = 0, ky != 1:            - S_row[r(ky)][D_x]      sums over one image row,    [N W] pixels
//   D_x = 0, kx != 1:            - S_col[q(kx)][D_y]      sums over one image column, [N H] pixels
//   D = 0, ky != 1 and kx != 1:  + K[r][q]                the corner pixel counted twice, [N] pixels
// 16 small matrices in all (2 rows x 3 shifts, 2 columns x 3 shifts, 4 corners).
//
// All 13 + 6 + 6 + 4 products are tiles of Gram matrices of "virtual" convolutions (stride 1, no padding at the top)
// and run on the direct-to-LDS tile of syrk_dtl_tile.hpp in ONE launch:
//   main    3 x 5 taps (dy = 0..2, dx = -2..2), positions = all pixels: rows [2C, 3C) (tap D = 0) times columns
//           [2C, 15C) (the 13 shifts (0,0..2), (1,-2..2), (2,-2..2)) of that Gram matrix;
//   rows    1 x 3 taps on the pixels of image row r;  columns  3 x 1 taps on the pixels of image column q;
//   corners 1 x 1 on the corner pixels.
// Every work group writes its accumulators as a partial tile; a second launch sums the partial tiles of the row
// splits in a fixed order into row-major matrices, a third assembles the dense factor in the (c, ky, kx) order,
// applying alpha and beta, with whole-line stores.  Executed matrix work: 26 M C^2 FLOP against 81 M C^2 for the
// upper triangle of U^T U.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <mutex>
#include <unordered_map>
#include "syrk_dtl_tile.hpp"

namespace ak {

constexpr int kCorrProds = 9;          // main, 2 image rows, 2 image columns, 4 corners
constexpr int kCorrShifts = 13;
constexpr int kCorrPieces = 29;        // [C, C] pieces of the reduced matrix: 13 shifts, 2 x 3 rows, 2 x 3 columns, 4 corners
constexpr int kCorrPiecesT = 25;       // of which the first 25 are also read transposed (the corners are symmetric)

struct CorrProd {
  const void* X;                       // first pixel of the product's positions
  int32_t M;                           // positions
  int32_t Ho, Wo, kw, KK, pw;          // virtual convolution (stride 1, no padding above)
  uint32_t mWo, mHo, mKw, mBlk;
  // Tiles: the row tap's C columns from tile ti0 on, `ntaps` column taps of C columns each from tile tj0 on.  With
  // an input of three bf16 planes (C = 3 c channels, [hi | mid | lo]) whose planes are whole tiles, only the six plane
  // pairs that matter are computed: npairs = 6, ppt = c / BT tiles per plane; else npairs = 1, ppt = C / BT.
  int32_t ti0, tj0, ntaps, ppt, npairs, tpt;    // tpt: tiles per tap in the column direction (C / BT)
  int32_t kt_split, nsplit;            // k-tiles per row split, splits
  int32_t first_item, first_tile;      // running counts over the products
  int64_t part_off;                    // float4 index of partial tile (split 0, tile 0)
  int64_t out_off;                     // first column of the product in the reduced matrix red[C][29 C]
};

struct CorrArgs {
  CorrProd prod[kCorrProds];
  int32_t Cin, H, W, nprod;
  uint32_t mG;
  floatx4* part;
  float* red;
};

__device__ __forceinline__ int corr_find(const CorrArgs& a, int w, bool by_tile) {
  int pi = 0;
#pragma unroll
  for (int i = 1; i < kCorrProds; ++i)
    if (i < a.nprod && w >= (by_tile ? a.prod[i].first_tile : a.prod[i].first_item)) pi = i;
  return pi;
}

// Tile t of a product: (ti, tj) in the virtual Gram matrix, and (row, col) = where the tile starts in the product's
// [C, ntaps C] block of the reduced matrix, in tiles.
__device__ __forceinline__ void corr_tile_of(const CorrProd& cp, int t, int& ti, int& tj, int& row, int& col) {
  const int per_pair = cp.ntaps * cp.ppt * cp.ppt;
  const int pair = t / per_pair, rem = t - pair * per_pair;
  const int tap = rem / (cp.ppt * cp.ppt), r2 = rem - tap * cp.ppt * cp.ppt;
  const int ii = r2 / cp.ppt, jj = r2 - ii * cp.ppt;
  // plane pairs in the order (0,0) (0,1) (0,2) (1,0) (1,1) (2,0): hi = 0, mid = 1, lo = 2, sum of the two <= 2
  const int pi = pair < 3 ? 0 : (pair < 5 ? 1 : 2), pj = pair < 3 ? pair : (pair < 5 ? pair - 3 : 0);
  row = pi * cp.ppt + ii;
  col = tap * cp.tpt + pj * cp.ppt + jj;
  ti = cp.ti0 + row;
  tj = cp.tj0 + col;
}

__device__ __forceinline__ int corr_ntiles(const CorrProd& cp) { return cp.npairs * cp.ntaps * cp.ppt * cp.ppt; }

// One work group per (product, row split, tile).
template <int WR, int WC, int FR, int FC>
__device__ __forceinline__ void corr_products_tile(const CorrArgs& a, uint32_t wg, uint32_t nwg) {
  constexpr int BT = DtlCfg<WR, WC, FR, FC, true>::BT;
  const int w = static_cast<int>(xcd_contiguous_id(wg, nwg));
  const CorrProd& cp = a.prod[corr_find(a, w, false)];
  DtlParams p{};
  p.X = cp.X;
  p.M = cp.M;
  p.d = static_cast<int64_t>(cp.KK) * a.Cin;
  p.Cin = a.Cin; p.H = a.H; p.W = a.W;
  p.kw = cp.kw; p.KK = cp.KK;
  p.sh = p.sw = 1; p.ph = 0; p.pw = cp.pw;
  p.Ho = cp.Ho; p.Wo = cp.Wo;
  p.G = a.Cin;
  p.mWo = cp.mWo; p.mHo = cp.mHo; p.mKw = cp.mKw; p.mBlk = cp.mBlk; p.mG = a.mG; p.mKK = 0;
  const int local = w - cp.first_item, ntiles = corr_ntiles(cp);
  const int s = local / ntiles, t = local - s * ntiles;
  int ti, tj, row, col;
  corr_tile_of(cp, t, ti, tj, row, col);
  const int64_t k_begin = static_cast<int64_t>(s) * cp.kt_split * kDtlBK;
  int64_t k_end = k_begin + static_cast<int64_t>(cp.kt_split) * kDtlBK;
  if (k_end > cp.M) k_end = cp.M;
  const int rows = k_begin < k_end ? static_cast<int>(k_end - k_begin) : 0;
  if (cp.nsplit == 1) {
    // the only split: the tile goes straight into the reduced matrix
    const int64_t ld = static_cast<int64_t>(kCorrPieces) * a.Cin;
    dtl_tile<WR, WC, FR, FC, true>(p, ti, tj, k_begin, rows, nullptr,
                                   a.red + cp.out_off + static_cast<int64_t>(row) * BT * ld + static_cast<int64_t>(col) * BT, ld);
    return;
  }
  floatx4* partial = a.part + cp.part_off + static_cast<int64_t>(local) * (BT * BT / 4);
  dtl_tile<WR, WC, FR, FC, true>(p, ti, tj, k_begin, rows, partial);
}

// Sums the partial tiles of the row splits (fixed order) into the product's columns of ONE row-major matrix
// red[C][29 C]: 13 C columns of the main product, 3 C per image row and image column, C per corner.
// grid (tiles of all products, 4 * FR * FC): one work group per float4 slot of every thread's accumulators.
template <int WR, int WC, int FR, int FC>
__device__ __forceinline__ void corr_reduce_tile(const CorrArgs& a, int tile, int slot) {
  constexpr int NW = WR * WC, BT = 32 * FR * WR;
  constexpr int64_t tile_f4 = BT * BT / 4;
  const CorrProd& cp = a.prod[corr_find(a, tile, true)];
  if (cp.nsplit == 1) return;                          // written by the product itself
  const int t = tile - cp.first_tile, ntiles = corr_ntiles(cp);
  int ti, tj, trow, tcol;
  corr_tile_of(cp, t, ti, tj, trow, tcol);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave / WC, wc = wave % WC, g = lane >> 5, l32 = lane & 31;
  const int q = slot & 3, b = (slot >> 2) % FC, aa = (slot >> 2) / FC;
  const floatx4* src = a.part + cp.part_off + t * tile_f4 + slot * (NW * 64) + tid;
  const int64_t stride = ntiles * tile_f4;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  int s = 0;
  for (; s + 8 <= cp.nsplit; s += 8) {                 // eight loads in flight, summed in order
    floatx4 w[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) w[k] = src[(s + k) * stride];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc += w[k];
  }
  for (; s < cp.nsplit; ++s) acc += src[s * stride];
  const int ld = kCorrPieces * a.Cin;
  const int row = trow * BT + 32 * FR * wr + 32 * aa + 8 * q + 4 * g;
  const int col = tcol * BT + 32 * FC * wc + 32 * b + l32;
  float* dst = a.red + cp.out_off + static_cast<int64_t>(row) * ld + col;
#pragma unroll
  for (int e = 0; e < 4; ++e) dst[static_cast<int64_t>(e) * ld] = acc[e];
}

// All products of one layer in one launch: one work group per (product, row split, tile).
template <int WR, int WC, int FR, int FC>
__global__ __launch_bounds__(WR * WC * 64) void corr_products_kernel(CorrArgs a) {
  corr_products_tile<WR, WC, FR, FC>(a, blockIdx.x, gridDim.x);
}

// grid (tiles of all products, 4 * FR * FC): one work group per float4 slot of every thread's accumulators.
template <int WR, int WC, int FR, int FC>
__global__ __launch_bounds__(WR * WC * 64) void corr_reduce_kernel(CorrArgs a) {
  corr_reduce_tile<WR, WC, FR, FC>(a, blockIdx.x, blockIdx.y);
}

// The dense factor from the reduced matrix.  One work group per block of CR channels of rows and 64 channels of
// columns: 9 CR x 576 elements.  A thread owns ONE result column (channel c2, tap t2) and walks down the rows, so
// a wave stores 64 consecutive floats of a row and the work group 576.  The [CR, 64] block of each of the 29 pieces
// and the [64, CR] block that the transposed shifts read are staged in the LDS first, all loads of a thread in
// flight at once.  For a fixed row tap t1 (a compile-time value in the unrolled loop) everything but the channel pair
// is a per-thread constant: which piece the element comes from, read straight or transposed, and which corrections
// apply.  Piece numbers: shift s = 5 dy + dx: s; image row e (0: first, 1: last), shift dx: 13 + 3 e + dx; image
// column e, shift dy: 19 + 3 e + dy; corner (r, q): 25 + 2 r + q.
struct CorrAsm {
  const float* red;
  float* A;
  int64_t lda;
  int32_t C;
  float alpha, beta;
};

constexpr int kAsmCC = 64;                      // channels of columns per work group
constexpr int kAsmThreads = 9 * kAsmCC;         // one thread per result column

template <int CR>
__global__ __launch_bounds__(kAsmThreads) void corr_assemble_kernel(CorrAsm a) {
  constexpr int FW = kAsmCC + 1, TW = CR + 1;            // row lengths of a straight / a transposed block
  constexpr int F = CR * FW, T = kAsmCC * TW;            // floats per block
  constexpr int SF = 0, ST = kCorrPieces * F;
  __shared__ float lds[kCorrPieces * F + kCorrPiecesT * T];
  const int tid = threadIdx.x, C = a.C;
  const int64_t ld = static_cast<int64_t>(kCorrPieces) * C;
  const int ci0 = blockIdx.y * CR, cj0 = blockIdx.x * kAsmCC;
  {
    // straight blocks: element (c1, c2) of piece pc is red[ci0 + c1][pc C + cj0 + c2]; consecutive threads read
    // consecutive c2.  transposed sources: red[cj0 + c2][pc C + ci0 + c1], consecutive threads consecutive c1.
    constexpr int NF = kCorrPieces * CR * kAsmCC, NT = kCorrPiecesT * CR * kAsmCC;
    constexpr int IF = (NF + kAsmThreads - 1) / kAsmThreads, IT = (NT + kAsmThreads - 1) / kAsmThreads;
    float vf[IF], vt[IT];
#pragma unroll
    for (int i = 0; i < IF; ++i) {
      const int idx = tid + i * kAsmThreads;
      const int c2 = idx % kAsmCC, c1 = (idx / kAsmCC) % CR, pc = idx / (kAsmCC * CR);
      vf[i] = idx < NF ? a.red[static_cast<int64_t>(ci0 + c1) * ld + pc * C + cj0 + c2] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const int idx = tid + i * kAsmThreads;
      const int c1 = idx % CR, c2 = (idx / CR) % kAsmCC, pc = idx / (kAsmCC * CR);
      vt[i] = idx < NT ? a.red[static_cast<int64_t>(cj0 + c2) * ld + pc * C + ci0 + c1] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < IF; ++i) {
      const int idx = tid + i * kAsmThreads;
      const int c2 = idx % kAsmCC, c1 = (idx / kAsmCC) % CR, pc = idx / (kAsmCC * CR);
      if (idx < NF) lds[SF + pc * F + c1 * FW + c2] = vf[i];
    }
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const int idx = tid + i * kAsmThreads;
      const int c1 = idx % CR, c2 = (idx / CR) % kAsmCC, pc = idx / (kAsmCC * CR);
      if (idx < NT) lds[ST + pc * T + c2 * TW + c1] = vt[i];
    }
  }
  __syncthreads();
  const int c2 = tid / 9, t2 = tid - 9 * c2, ky2 = t2 / 3, kx2 = t2 - 3 * ky2;
  float* dst = a.A + static_cast<int64_t>(ci0) * 9 * a.lda + static_cast<int64_t>(cj0) * 9 + tid;
  // where element (c1, this thread's c2) of piece pc lies: straight, or in the transposed block
  auto at_of = [&](int pc, bool straight, int& stride) {
    stride = straight ? FW : 1;
    return straight ? SF + pc * F + c2 : ST + pc * T + c2 * TW;
  };
#pragma unroll
  for (int t1 = 0; t1 < 9; ++t1) {
    const int ky = t1 / 3, kx = t1 % 3;
    const int dy = ky2 - ky, dx = kx2 - kx, s = dy * 5 + dx;
    const int adx = dx >= 0 ? dx : -dx, ady = dy >= 0 ? dy : -dy;
    // main term: shift s >= 0 is stored, s < 0 is the transpose of shift -s
    int m_st, r_st = 0, c_st = 0;
    const int m_at = at_of(s >= 0 ? s : -s, s >= 0, m_st);
    // corrections: the pixels of one image row / column have no output position under this row tap
    const int r = ky == 0 ? 1 : 0, q = kx == 0 ? 1 : 0;
    const bool use_r = ky != 1 && dy == 0, use_c = kx != 1 && dx == 0, use_k = ky != 1 && kx != 1 && s == 0;
    const int r_at = use_r ? at_of(13 + 3 * r + adx, dx >= 0, r_st) : 0;     // unused: a dummy read of lds[0]
    const int c_at = use_c ? at_of(19 + 3 * q + ady, dy >= 0, c_st) : 0;
    const int k_at = SF + (25 + 2 * r + q) * F + c2;
#pragma unroll
    for (int c1 = 0; c1 < CR; ++c1) {
      float v = lds[m_at + c1 * m_st];
      if (ky != 1) { const float x = lds[r_at + c1 * r_st]; v -= use_r ? x : 0.f; }
      if (kx != 1) { const float x = lds[c_at + c1 * c_st]; v -= use_c ? x : 0.f; }
      if (ky != 1 && kx != 1) { const float x = lds[k_at + c1 * FW]; v += use_k ? x : 0.f; }
      float* o = dst + static_cast<int64_t>(c1 * 9 + t1) * a.lda;
      v *= a.alpha;
      if (a.beta != 0.f) v += a.beta * *o;
      *o = v;
    }
  }
}

// ---- fp32 inputs: three bf16 planes ------------------------------------------------------------------------------
// An fp32 NCHW input takes the same path on the bf16 matrix cores at the accuracy of fp32 products: every element
// is split exactly into three bf16 pieces, x = hi + mid + lo (each the remainder rounded to the nearest bf16; the
// third needs no rounding), written as a channels-last tensor with 3 C channels, [hi | mid | lo] per pixel.  The
// products above then run on that tensor as they are (3 C channels), and before the assembly the 3 x 3 blocks of
// every [3 C, 3 C] piece are folded into [C, C]:  x^T y ~= hi^T hi' + (hi^T mid' + mid^T hi') + (hi^T lo' + lo^T hi')
// + mid^T mid'; the three dropped blocks are below 2^-24 of the product.  The pairs are added in this order so that
// the fold of a symmetric piece is symmetric to the last bit.

// x: [N, C, HW] fp32 (HW contiguous) -> planes: [N, HW, 3 C] bf16.  One work group per (sample, 32 pixels, 32
// channels): coalesced 128-byte reads along the pixels, 64-byte runs of channels per pixel and plane on the way out.
__global__ __launch_bounds__(256) void corr_split_nchw_kernel(const float* __restrict__ x, uint16_t* __restrict__ planes,
                                                              int C, int HW) {
  __shared__ float tile[32][33];
  const int n = blockIdx.z, p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;          // 32 x 8
  const float* src = x + (static_cast<int64_t>(n) * C + c0) * HW + p0;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int c = ty + 8 * r;
    tile[c][tx] = p0 + tx < HW ? src[static_cast<int64_t>(c) * HW + tx] : 0.f;
  }
  __syncthreads();
  uint16_t* dst = planes + (static_cast<int64_t>(n) * HW + p0) * (3 * C) + c0;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int px = ty + 8 * r;
    if (p0 + px >= HW) continue;
    const float v = tile[tx][px];
    const __bf16 hi = static_cast<__bf16>(v);
    const float r1 = v - static_cast<float>(hi);
    const __bf16 mid = static_cast<__bf16>(r1);
    const __bf16 lo = static_cast<__bf16>(r1 - static_cast<float>(mid));
    uint16_t* q = dst + static_cast<int64_t>(px) * (3 * C) + tx;
    q[0] = __builtin_bit_cast(uint16_t, hi);
    q[C] = __builtin_bit_cast(uint16_t, mid);
    q[2 * C] = __builtin_bit_cast(uint16_t, lo);
  }
}

// red3: [3 C][29 * 3 C] (pieces of 3 C columns) -> red: [C][29 * C].  grid (29 C / 256, C).
__global__ __launch_bounds__(256) void corr_fold_kernel(const float* __restrict__ red3, float* __restrict__ red, int C) {
  const int col = blockIdx.x * 256 + threadIdx.x, c = blockIdx.y;
  if (col >= kCorrPieces * C) return;
  const int pc = col / C, c2 = col - pc * C;
  const int64_t ld3 = static_cast<int64_t>(kCorrPieces) * 3 * C;
  auto at = [&](int p, int q) { return red3[static_cast<int64_t>(p * C + c) * ld3 + pc * 3 * C + q * C + c2]; };
  const float hh = at(0, 0), hm = at(0, 1) + at(1, 0), hl = at(0, 2) + at(2, 0), mm = at(1, 1);
  red[static_cast<int64_t>(c) * (kCorrPieces * C) + col] = ((hh + hm) + hl) + mm;
}

// ---- host side ------------------------------------------------------------------------------------------------

struct CorrPlan {
  CorrArgs args;            // X pointers, part and red are filled in per call
  int bt, items, tiles;
  size_t part_f4, red_floats;
  int64_t x_off[kCorrProds];   // byte offset of each product's first pixel from the tensor
};

static int corr_tile_width(int64_t C) {
  if (C % 256 == 0 && C >= 512) return 256;
  if (C % 128 == 0) return 128;
  if (C % 192 == 0) return 192;
  if (C % 64 == 0) return 64;
  return 0;
}

// ASDL_AMD_CONV_CORR=0 in the environment keeps the unfolded form for every layer (read once).
static bool corr_enabled() {
  static const bool on = [] {
    const char* v = std::getenv("ASDL_AMD_CONV_CORR");
    return !(v != nullptr && v[0] == '0');
  }();
  return on;
}

static bool corr_eligible(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw) {
  if (!corr_enabled()) return false;
  if (kh != 3 || kw != 3 || sh != 1 || sw != 1 || ph != 1 || pw != 1) return false;
  if (corr_tile_width(C) == 0 || N <= 0 || H <= 0 || W <= 0) return false;
  if (N * H * W * C * 2 > static_cast<int64_t>(kDtlRange)) return false;          // 32-bit byte offsets
  if (N * H * W * (W > H ? W : H) >= (1ll << 32)) return false;                   // exact magic divisions
  if (15 * C * (15 * C + 256) >= (1ll << 32)) return false;
  return true;
}

// planes: 1, or 3 when the C channels are the three bf16 planes of C / 3 channels
static CorrPlan corr_plan_build(int64_t N, int64_t C, int64_t H, int64_t W, int planes) {
  CorrPlan pl{};
  const int bt = corr_tile_width(C);
  pl.bt = bt;
  const int cb = static_cast<int>(C / bt);
  // the unneeded plane pairs can be left out when every plane is a whole number of tiles
  const bool pairs = planes == 3 && (C / 3) % bt == 0;
  const int occ = bt == 64 ? 4 : (bt == 128 ? 2 : 1);      // work groups per CU
  const int64_t slots = 256 * occ;
  CorrArgs& a = pl.args;
  a.Cin = static_cast<int32_t>(C); a.H = static_cast<int32_t>(H); a.W = static_cast<int32_t>(W);
  a.nprod = kCorrProds;
  a.mG = make_magic(static_cast<uint32_t>(C));
  auto fill = [&](int i, int64_t x_off, int64_t M, int64_t Ho, int64_t Wo, int kh_v, int kw_v, int pw_v, int ti0,
                  int tj0, int ntaps) {
    CorrProd& p = a.prod[i];
    pl.x_off[i] = x_off;
    p.M = static_cast<int32_t>(M);
    p.Ho = static_cast<int32_t>(Ho); p.Wo = static_cast<int32_t>(Wo);
    p.kw = kw_v; p.KK = kh_v * kw_v; p.pw = pw_v;
    p.mWo = make_magic(p.Wo); p.mHo = make_magic(p.Ho); p.mKw = make_magic(kw_v);
    p.mBlk = make_magic(static_cast<uint32_t>(C) * p.KK);
    p.ti0 = ti0; p.tj0 = tj0; p.ntaps = ntaps;
    p.tpt = cb;
    p.npairs = pairs ? 6 : 1;
    p.ppt = pairs ? cb / 3 : cb;
  };
  const int64_t px = C * 2;                      // bytes per pixel
  fill(0, 0, N * H * W, H, W, 3, 5, 2, 2 * cb, 2 * cb, kCorrShifts);
  fill(1, 0, N * W, 1, W, 1, 3, 0, 0, 0, 3);                         // image row 0
  fill(2, (H - 1) * W * px, N * W, 1, W, 1, 3, 0, 0, 0, 3);          // image row H - 1
  fill(3, 0, N * H, H, 1, 3, 1, 0, 0, 0, 3);                         // image column 0
  fill(4, (W - 1) * px, N * H, H, 1, 3, 1, 0, 0, 0, 3);              // image column W - 1
  for (int r = 0; r < 2; ++r)
    for (int q = 0; q < 2; ++q)
      fill(5 + 2 * r + q, ((r ? H - 1 : 0) * W + (q ? W - 1 : 0)) * px, N, 1, 1, 1, 1, 0, 0, 0, 1);
  int items = 0, tiles = 0;
  size_t part = 0;
  int64_t red_col = 0;
  const size_t tile_f4 = static_cast<size_t>(bt) * bt / 4;
  for (int i = 0; i < kCorrProds; ++i) {
    CorrProd& p = a.prod[i];
    const int64_t ktiles = (p.M + kDtlBK - 1) / kDtlBK,
                  ntiles = static_cast<int64_t>(p.npairs) * p.ntaps * p.ppt * p.ppt;
    int64_t ns = 1;
    if (i == 0 && ntiles > 0) {
      // the main product fills the device once (the corrections ride in its tail); at least 8 k-tiles per split
      ns = (slots + ntiles / 2) / ntiles;
      const int64_t cap = ktiles / 8 < 1 ? 1 : ktiles / 8;
      if (ns > cap) ns = cap;
      if (ns < 1) ns = 1;
    } else if (i > 0) {
      ns = (ktiles + 15) / 16;          // corrections: chains of at most 16 k-tiles
    }
    p.kt_split = static_cast<int32_t>((ktiles + ns - 1) / ns);
    p.nsplit = static_cast<int32_t>((ktiles + p.kt_split - 1) / p.kt_split);
    p.first_item = items;
    p.first_tile = tiles;
    p.part_off = static_cast<int64_t>(part);
    p.out_off = red_col;
    red_col += static_cast<int64_t>(p.ntaps) * C;      // C per piece: 13 C, 3 C or C
    items += p.nsplit * static_cast<int>(ntiles);
    tiles += static_cast<int>(ntiles);
    part += static_cast<size_t>(p.nsplit) * ntiles * tile_f4;
  }
  pl.items = items;
  pl.tiles = tiles;
  pl.part_f4 = part;
  pl.red_floats = static_cast<size_t>(C) * kCorrPieces * C;       // red_col == 29 C
  return pl;
}

static CorrPlan corr_plan(int64_t N, int64_t C, int64_t H, int64_t W, int planes = 1) {
  struct Key {
    int64_t N, C, H, W;
    bool operator==(const Key& o) const { return N == o.N && C == o.C && H == o.H && W == o.W; }
  };
  H = planes == 3 ? -H : H;      // the two kinds of plan for one shape are two cache entries
  struct Hash {
    size_t operator()(const Key& k) const {
      uint64_t h = 0x9e3779b97f4a7c15ull;
      for (uint64_t v : {static_cast<uint64_t>(k.N), static_cast<uint64_t>(k.C), static_cast<uint64_t>(k.H),
                         static_cast<uint64_t>(k.W)})
        h = (h ^ v) * 0xff51afd7ed558ccdull + (h >> 29);
      return static_cast<size_t>(h);
    }
  };
  static std::unordered_map<Key, CorrPlan, Hash> cache;
  static std::mutex lock;
  const Key key{N, C, H, W};
  std::lock_guard<std::mutex> guard(lock);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  if (cache.size() > 1024) cache.clear();
  const CorrPlan plan = corr_plan_build(N, C, H < 0 ? -H : H, W, planes);
  cache.emplace(key, plan);
  return plan;
}

static size_t corr_ws_layout(const CorrPlan& pl, size_t& red_at) {
  const size_t part_bytes = pl.part_f4 * sizeof(floatx4);
  red_at = (part_bytes + 255) & ~static_cast<size_t>(255);
  return red_at + pl.red_floats * sizeof(float);
}

template <int WR, int WC, int FR, int FC>
static int corr_launch_cfg(const CorrPlan& pl, const CorrArgs& args, hipStream_t stream) {
  using Cfg = DtlCfg<WR, WC, FR, FC, true>;
  auto kern = corr_products_kernel<WR, WC, FR, FC>;
  if (Cfg::LDS_BYTES > 64 * 1024) {
    static bool attr_set = false;     // idempotent; a race sets it twice at worst
    if (!attr_set) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              Cfg::LDS_BYTES) != hipSuccess)
        return AK_ERR_LAUNCH;
      attr_set = true;
    }
  }
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(pl.items)), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, stream, args);
  hipLaunchKernelGGL((corr_reduce_kernel<WR, WC, FR, FC>), dim3(static_cast<unsigned>(pl.tiles), 4 * FR * FC),
                     dim3(Cfg::NW * 64), 0, stream, args);
  return AK_OK;
}

size_t conv_corr_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw) {
  if (!corr_eligible(N, C, H, W, kh, kw, sh, sw, ph, pw)) return 0;
  size_t red_at;
  return corr_ws_layout(corr_plan(N, C, H, W), red_at);
}

// All products of the layer on the channels-last bf16 tensor x (C channels), reduced into red [C][29 C].
static int corr_products(const CorrPlan& plan, const void* x, floatx4* part, float* red, hipStream_t stream) {
  CorrPlan pl = plan;
  CorrArgs& args = pl.args;
  for (int i = 0; i < kCorrProds; ++i) args.prod[i].X = static_cast<const unsigned char*>(x) + pl.x_off[i];
  args.part = part;
  args.red = red;
  if (pl.bt == 64) return corr_launch_cfg<2, 2, 1, 1>(pl, args, stream);
  if (pl.bt == 128) return corr_launch_cfg<2, 2, 2, 2>(pl, args, stream);
  if (pl.bt == 192) return corr_launch_cfg<2, 2, 3, 3>(pl, args, stream);
  return corr_launch_cfg<2, 4, 4, 2>(pl, args, stream);
}

static int corr_assemble(const float* red, int64_t C, float alpha, float beta, float* A, int64_t lda, hipStream_t stream) {
  CorrAsm s{};
  s.red = red;
  s.A = A; s.lda = lda;
  s.C = static_cast<int32_t>(C);
  s.alpha = alpha; s.beta = beta;
  // channels of rows per work group: 4 (60 KB of LDS) where that still gives a work group per CU
  const dim3 block(kAsmThreads);
  if (C >= 256)
    hipLaunchKernelGGL((corr_assemble_kernel<4>), dim3(static_cast<unsigned>(C / kAsmCC), static_cast<unsigned>(C / 4)),
                       block, 0, stream, s);
  else if (C >= 128)
    hipLaunchKernelGGL((corr_assemble_kernel<2>), dim3(static_cast<unsigned>(C / kAsmCC), static_cast<unsigned>(C / 2)),
                       block, 0, stream, s);
  else
    hipLaunchKernelGGL((corr_assemble_kernel<1>), dim3(static_cast<unsigned>(C / kAsmCC), static_cast<unsigned>(C)),
                       block, 0, stream, s);
  return check_launch();
}

int conv_corr_syrk(const void* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                   int pw, float alpha, float beta, float* A, int64_t lda, void* ws, size_t ws_bytes,
                   hipStream_t stream) {
  if (!corr_eligible(N, C, H, W, kh, kw, sh, sw, ph, pw) || (reinterpret_cast<uintptr_t>(x) & 15) != 0)
    return AK_ERR_UNSUPPORTED;
  const CorrPlan pl = corr_plan(N, C, H, W);
  size_t red_at;
  const size_t need = corr_ws_layout(pl, red_at);
  if (ws == nullptr || ws_bytes < need) return AK_ERR_WORKSPACE;
  float* red = reinterpret_cast<float*>(static_cast<unsigned char*>(ws) + red_at);
  const int rc = corr_products(pl, x, static_cast<floatx4*>(ws), red, stream);
  if (rc != AK_OK) return rc;
  return corr_assemble(red, C, alpha, beta, A, lda, stream);
}

// fp32 NCHW input: [planes: N H W 3C bf16][workspace of the 3 C-channel products, its reduced matrix last][red: C x 29 C]
static size_t corr_f32_layout(int64_t N, int64_t C, int64_t H, int64_t W, const CorrPlan& pl3, size_t& ws3_at,
                              size_t& red3_in_ws3, size_t& red_at) {
  const size_t planes = static_cast<size_t>(N) * H * W * 3 * C * 2;
  ws3_at = (planes + 255) & ~static_cast<size_t>(255);
  const size_t ws3 = corr_ws_layout(pl3, red3_in_ws3);
  red_at = (ws3_at + ws3 + 255) & ~static_cast<size_t>(255);
  return red_at + static_cast<size_t>(C) * kCorrPieces * C * sizeof(float);
}

size_t conv_corr_f32_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw) {
  if (C % 64 != 0 || !corr_eligible(N, 3 * C, H, W, kh, kw, sh, sw, ph, pw)) return 0;
  size_t a, b, c;
  return corr_f32_layout(N, C, H, W, corr_plan(N, 3 * C, H, W, 3), a, b, c);
}

int conv_corr_syrk_f32(const float* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                       int pw, float alpha, float beta, float* A, int64_t lda, void* ws, size_t ws_bytes,
                       hipStream_t stream) {
  if (C % 64 != 0 || !corr_eligible(N, 3 * C, H, W, kh, kw, sh, sw, ph, pw)) return AK_ERR_UNSUPPORTED;
  const CorrPlan pl3 = corr_plan(N, 3 * C, H, W, 3);
  size_t ws3_at, red3_in_ws3, red_at;
  const size_t need = corr_f32_layout(N, C, H, W, pl3, ws3_at, red3_in_ws3, red_at);
  if (ws == nullptr || ws_bytes < need || (reinterpret_cast<uintptr_t>(ws) & 255) != 0) return AK_ERR_WORKSPACE;
  unsigned char* base = static_cast<unsigned char*>(ws);
  uint16_t* planes = reinterpret_cast<uint16_t*>(base);
  const int HW = static_cast<int>(H * W);
  hipLaunchKernelGGL(corr_split_nchw_kernel, dim3((HW + 31) / 32, static_cast<unsigned>(C / 32), static_cast<unsigned>(N)),
                     dim3(256), 0, stream, x, planes, static_cast<int>(C), HW);
  float* red3 = reinterpret_cast<float*>(base + ws3_at + red3_in_ws3);
  const int rc = corr_products(pl3, planes, reinterpret_cast<floatx4*>(base + ws3_at), red3, stream);
  if (rc != AK_OK) return rc;
  float* red = reinterpret_cast<float*>(base + red_at);
  hipLaunchKernelGGL(corr_fold_kernel, dim3(static_cast<unsigned>((kCorrPieces * C + 255) / 256), static_cast<unsigned>(C)),
                     dim3(256), 0, stream, red3, red, static_cast<int>(C));
  return corr_assemble(red, C, alpha, beta, A, lda, stream);
}

}  // namespace ak
