// Host side and launch kernels of the direct-to-LDS bf16 rank-k update (device side: syrk_dtl_tile.hpp).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <initializer_list>
#include <functional>
#include <mutex>
#include <queue>
#include <unordered_map>
#include <vector>
#include <type_traits>
#include "syrk_dtl_tile.hpp"

namespace ak {

// One factor per launch: grid (upper tiles, splits).
template <int WR, int WC, int FR, int FC, bool GATHER>
__global__ __launch_bounds__(WR * WC * 64) void syrk_dtl_kernel(DtlParams p) {
  constexpr int BT = DtlCfg<WR, WC, FR, FC, GATHER>::BT;
  const uint32_t logical = xcd_contiguous_id(blockIdx.x + blockIdx.y * gridDim.x, gridDim.x * gridDim.y);
  const uint32_t split_id = logical / gridDim.x, tile_id = logical - split_id * gridDim.x;
  int ti, tj;
  decode_upper_tile(tile_id, p.T, ti, tj);
  const int64_t k_begin = static_cast<int64_t>(split_id) * p.rows_per_split;
  int64_t k_end = k_begin + p.rows_per_split;
  if (k_end > p.M) k_end = p.M;
  const int rows = k_begin < k_end ? static_cast<int>(k_end - k_begin) : 0;
  floatx4* partial = nullptr;
  if (p.nsplit > 1)
    partial = reinterpret_cast<floatx4*>(p.ws) + (static_cast<size_t>(split_id) * gridDim.x + tile_id) * (BT * BT / 4);
  dtl_tile<WR, WC, FR, FC, GATHER>(p, ti, tj, k_begin, rows, partial);
}

// Many factors per launch.  Work item w (device table): a tile of a factor and a range of its rows.  The items of
// one (factor, split) are adjacent, so the renumbering above still gives them one L2.
struct DtlGroupItem {
  int32_t factor, tile;
  int32_t k_begin_tile, k_tiles;   // in k-tiles of kDtlBK rows
  int64_t partial;                 // float4 index into the workspace, or -1: this item is the whole sum
};

template <int WR, int WC, int FR, int FC, bool GATHER>
__global__ __launch_bounds__(WR * WC * 64) void syrk_dtl_grouped_kernel(const DtlParams* __restrict__ factors,
                                                                        const DtlGroupItem* __restrict__ items,
                                                                        floatx4* __restrict__ ws) {
  const DtlGroupItem it = items[xcd_contiguous_id(blockIdx.x, gridDim.x)];
  const DtlParams p = factors[it.factor];
  int ti, tj;
  decode_upper_tile(it.tile, p.T, ti, tj);
  const int64_t k_begin = static_cast<int64_t>(it.k_begin_tile) * kDtlBK;
  int64_t k_end = k_begin + static_cast<int64_t>(it.k_tiles) * kDtlBK;
  if (k_end > p.M) k_end = p.M;
  const int rows = k_begin < k_end ? static_cast<int>(k_end - k_begin) : 0;
  dtl_tile<WR, WC, FR, FC, GATHER>(p, ti, tj, k_begin, rows, it.partial >= 0 ? ws + it.partial : nullptr);
}

// Split-K reduction, first stage (only for many splits): work group (tile, slot, g) sums partials
// [g*group, min((g+1)*group, n)) of its float4 slot and writes the sum as partial g of a second buffer with
// the same layout.  Fixed summation order.
template <int NT>
__global__ __launch_bounds__(NT) void syrk_dtl_reduce_kernel(const floatx4* __restrict__ src, floatx4* __restrict__ dst,
                                                             int n, int group, size_t tile_f4) {
  const size_t split_stride = static_cast<size_t>(gridDim.x) * tile_f4;
  const size_t off = blockIdx.x * tile_f4 + static_cast<size_t>(blockIdx.y) * NT + threadIdx.x;
  const int s0 = blockIdx.z * group;
  const int s1 = s0 + group < n ? s0 + group : n;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  int s = s0;
  for (; s + 4 <= s1; s += 4) {
    const floatx4 w0 = src[off + (s + 0) * split_stride], w1 = src[off + (s + 1) * split_stride];
    const floatx4 w2 = src[off + (s + 2) * split_stride], w3 = src[off + (s + 3) * split_stride];
    acc += w0; acc += w1; acc += w2; acc += w3;
  }
  for (; s < s1; ++s) acc += src[off + s * split_stride];
  dst[off + blockIdx.z * split_stride] = acc;
}

// Sums n partial tiles (split_stride float4 apart) of tile (ti, tj) in a fixed order and applies the epilogue; one
// work group per float4 slot (a, b, q) of every thread's accumulators.
template <int WR, int WC, int FR, int FC, bool GATHER>
__device__ __forceinline__ void dtl_finalize_slot(const DtlParams& p, int ti, int tj, int slot,
                                                  const floatx4* __restrict__ tile_part, size_t split_stride, int n) {
  constexpr int NW = WR * WC, BT = 32 * FR * WR;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave / WC, wc = wave % WC, g = lane >> 5, l32 = lane & 31;
  const int q = slot & 3, b = (slot >> 2) % FC, a = (slot >> 2) / FC;
  const floatx4* src = tile_part + slot * (NW * 64) + tid;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  int s = 0;
  for (; s + 4 <= n; s += 4) {
    const floatx4 w0 = src[(s + 0) * split_stride], w1 = src[(s + 1) * split_stride];
    const floatx4 w2 = src[(s + 2) * split_stride], w3 = src[(s + 3) * split_stride];
    acc += w0; acc += w1; acc += w2; acc += w3;
  }
  for (; s < n; ++s) acc += src[s * split_stride];
  const int64_t gj = static_cast<int64_t>(tj) * BT + 32 * FC * wc + 32 * b + l32;
  const int64_t gi = static_cast<int64_t>(ti) * BT + 32 * FR * wr + 32 * a + 8 * q + 4 * g;
  if (gj >= p.d) return;
  const int64_t oj = out_index<GATHER>(gj, p);
  int64_t oi[4];
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {                    // rows beyond d are clamped for the reads and skipped by the stores
    oi[e] = out_index<GATHER>(gi + e < p.d ? gi + e : p.d - 1, p);
    v[e] = p.alpha * acc[e];
  }
  if (p.beta != 0.f) {                             // all reads of C before any store to it, none under a condition
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += p.beta * p.C[oi[e] * p.ldc + oj];
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (gi + e >= p.d) continue;
    p.C[oi[e] * p.ldc + oj] = v[e];
    if (ti != tj) p.C[oj * p.ldc + oi[e]] = v[e];
  }
}

// grid (tiles, 4*FR*FC)
template <int WR, int WC, int FR, int FC, bool GATHER>
__global__ __launch_bounds__(WR * WC * 64) void syrk_dtl_finalize_kernel(DtlParams p, const floatx4* __restrict__ part,
                                                                         int n) {
  constexpr int BT = 32 * FR * WR;
  int ti, tj;
  decode_upper_tile(blockIdx.x, p.T, ti, tj);
  const size_t tile_f4 = BT * BT / 4;
  dtl_finalize_slot<WR, WC, FR, FC, GATHER>(p, ti, tj, blockIdx.y, part + blockIdx.x * tile_f4,
                                            static_cast<size_t>(gridDim.x) * tile_f4, n);
}

// The reduction pass of a grouped launch: grid (split tiles of all factors, 4*FR*FC).
struct DtlGroupFin {
  int32_t factor, tile, nparts, pad;
  int64_t first, stride;           // float4 index of the first partial of the tile, distance to the next one
};

template <int WR, int WC, int FR, int FC, bool GATHER>
__global__ __launch_bounds__(WR * WC * 64) void syrk_dtl_finalize_grouped_kernel(const DtlParams* __restrict__ factors,
                                                                                 const DtlGroupFin* __restrict__ fins,
                                                                                 const floatx4* __restrict__ ws) {
  const DtlGroupFin it = fins[blockIdx.x];
  const DtlParams p = factors[it.factor];
  int ti, tj;
  decode_upper_tile(it.tile, p.T, ti, tj);
  dtl_finalize_slot<WR, WC, FR, FC, GATHER>(p, ti, tj, blockIdx.y, ws + it.first, static_cast<size_t>(it.stride),
                                            it.nparts);
}

// Reduction pass of a GATHERED factor by output position.  The pass above takes the partial tiles in accumulator
// order, whose neighbouring columns are KK floats apart in the result (working order (c/G, tap, c%G), result order
// (c, tap)): every lane stores 4 bytes here and 4 bytes there, and the memory system writes 7 bytes for each one
// stored.  Here a wave owns four result rows, (c .. c+3, tap) for a channel quad c, and 64 consecutive result
// columns: its stores are whole 256-byte runs.  The four rows are consecutive working rows, i.e. ONE float4 of a
// partial tile, if the element lies in a computed (upper) tile; below the diagonal the mirror image is read, four
// floats from four float4.  grid (ceil(d / 64), ceil(d / 16)), 256 threads.
template <int WR, int WC, int FR, int FC>
__device__ __forceinline__ void dtl_finalize_out(const DtlParams& p, const floatx4* __restrict__ part, int64_t ntiles,
                                                 int n, uint32_t col_block, uint32_t row_block) {
  constexpr int NW = WR * WC, BT = 32 * FR * WR;
  constexpr size_t tile_f4 = static_cast<size_t>(BT) * BT / 4;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t d = static_cast<uint32_t>(p.d), KK = p.KK, G = p.G;
  const uint32_t oj = col_block * 64 + lane;
  const uint32_t rg = row_block * 4 + wave;                 // row group: (channel quad, tap)
  if (rg * 4 >= d || oj >= d) return;
  const uint32_t c4 = fastdiv(rg, p.mKK, KK), tap_i = rg - c4 * KK, ci = 4 * c4;
  const uint32_t blk_i = fastdiv(ci, p.mG, G);
  const uint32_t vi = blk_i * G * KK + tap_i * G + (ci - blk_i * G);      // first of four consecutive working rows
  const uint32_t cj = fastdiv(oj, p.mKK, KK), tap_j = oj - cj * KK, blk_j = fastdiv(cj, p.mG, G);
  const uint32_t vj = blk_j * G * KK + tap_j * G + (cj - blk_j * G);
  const uint32_t ti = vi / BT, tj = vj / BT;
  // float4 index and component of element (r, c) of a tile, in accumulator order
  auto slot_of = [](uint32_t r, uint32_t c, uint32_t& e) {
    const uint32_t wr = r / (32 * FR), a = (r % (32 * FR)) / 32, r32 = r % 32, q = r32 / 8, g = (r32 % 8) / 4;
    const uint32_t wc = c / (32 * FC), b = (c % (32 * FC)) / 32, l32 = c % 32;
    e = r32 % 4;
    return ((a * FC + b) * 4 + q) * (NW * 64) + (wr * WC + wc) * 64 + g * 32 + l32;
  };
  const size_t split_stride = static_cast<size_t>(ntiles) * tile_f4;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  if (ti <= tj) {
    const size_t tile = static_cast<size_t>(ti) * p.T - static_cast<size_t>(ti) * (ti - 1) / 2 + (tj - ti);
    uint32_t e;
    const floatx4* src = part + tile * tile_f4 + slot_of(vi % BT, vj % BT, e);     // e == 0: vi is a multiple of 4
    int s = 0;
    for (; s + 4 <= n; s += 4) {
      const floatx4 w0 = src[(s + 0) * split_stride], w1 = src[(s + 1) * split_stride];
      const floatx4 w2 = src[(s + 2) * split_stride], w3 = src[(s + 3) * split_stride];
      acc += w0; acc += w1; acc += w2; acc += w3;
    }
    for (; s < n; ++s) acc += src[s * split_stride];
  } else {
    const size_t tile = static_cast<size_t>(tj) * p.T - static_cast<size_t>(tj) * (tj - 1) / 2 + (ti - tj);
    const float* base = reinterpret_cast<const float*>(part + tile * tile_f4);
    size_t off[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      uint32_t e;
      const uint32_t f4 = slot_of(vj % BT, (vi + k) % BT, e);
      off[k] = static_cast<size_t>(f4) * 4 + e;
    }
    for (int s = 0; s < n; ++s) {
      const float* q = base + static_cast<size_t>(s) * split_stride * 4;
      const float x0 = q[off[0]], x1 = q[off[1]], x2 = q[off[2]], x3 = q[off[3]];
      acc[0] += x0; acc[1] += x1; acc[2] += x2; acc[3] += x3;
    }
  }
  float* dst = p.C + (static_cast<int64_t>(ci) * KK + tap_i) * p.ldc + oj;       // rows are KK apart
  const int64_t row_step = static_cast<int64_t>(KK) * p.ldc;
  float v[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) v[k] = p.alpha * acc[k];
  if (p.beta != 0.f) {
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] += p.beta * dst[k * row_step];
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) dst[k * row_step] = v[k];
}

template <int WR, int WC, int FR, int FC>
__global__ __launch_bounds__(256) void syrk_dtl_finalize_out_kernel(DtlParams p, const floatx4* __restrict__ part,
                                                                    int64_t ntiles, int n) {
  dtl_finalize_out<WR, WC, FR, FC>(p, part, ntiles, n, blockIdx.x, blockIdx.y);
}

// The same reduction, staged through the LDS: every partial tile is read with whole-line float4 loads and every
// result line is stored whole, the mirror image included.  The permutation between the working order and the result
// order stays inside a channel group of G * KK columns, so a work group takes four channels of rows (4 * KK result
// rows: KK float4 rows of the partial tiles) and cpb channels of columns (cpb * KK result columns, cpb a divisor of
// G), sums its float4 over the splits, scatters them into an LDS block in result order and stores the block row by
// row.  Column blocks in a channel group right of the rows' group also store the transposed block (runs of 4 * KK
// floats); blocks in the rows' own group are each computed by their own work group (elements whose tile lies below
// the diagonal read the mirror image, four floats), blocks left of it are those transposed stores.
// grid (Cin / cpb, Cin / 4), 256 threads, 4 * KK * (cpb * KK + 1) floats of LDS.
template <int WR, int WC, int FR, int FC>
__global__ __launch_bounds__(256) void syrk_dtl_finalize_blk_kernel(DtlParams p, const floatx4* __restrict__ part,
                                                                    int64_t ntiles, int n, int cpb) {
  constexpr int NW = WR * WC, BT = 32 * FR * WR;
  constexpr size_t tile_f4 = static_cast<size_t>(BT) * BT / 4;
  extern __shared__ float blk_lds[];
  const uint32_t tid = threadIdx.x;
  const uint32_t KK = p.KK, G = p.G, GKK = G * KK;
  const uint32_t ci0 = blockIdx.y * 4, cj0 = blockIdx.x * cpb;          // first channel of the rows / of the columns
  const uint32_t grp_i = fastdiv(ci0, p.mG, G), grp_j = fastdiv(cj0, p.mG, G);
  if (grp_j < grp_i) return;
  const uint32_t cols = cpb * KK, rows = 4 * KK, lw = cols + 1;
  auto slot_of = [](uint32_t r, uint32_t c, uint32_t& e) {
    const uint32_t wr = r / (32 * FR), a = (r % (32 * FR)) / 32, r32 = r % 32, q = r32 / 8, g = (r32 % 8) / 4;
    const uint32_t wc = c / (32 * FC), b = (c % (32 * FC)) / 32, l32 = c % 32;
    e = r32 % 4;
    return ((a * FC + b) * 4 + q) * (NW * 64) + (wr * WC + wc) * 64 + g * 32 + l32;
  };
  const size_t split_stride = static_cast<size_t>(ntiles) * tile_f4;
  const uint32_t vi_base = grp_i * GKK + (ci0 - grp_i * G), vj_base = grp_j * GKK + (cj0 - grp_j * G);
  for (uint32_t item = tid; item < KK * cols; item += 256) {
    const uint32_t tap_i = item / cols, idx = item - tap_i * cols;
    const uint32_t vi = vi_base + tap_i * G;                              // four consecutive working rows
    const uint32_t ti = vi / BT;
    {
      const uint32_t tap_j = idx / cpb, cgl = idx - tap_j * cpb;
      const uint32_t vj = vj_base + tap_j * G + cgl;
      const uint32_t tj = vj / BT;
      floatx4 acc = {0.f, 0.f, 0.f, 0.f};
      if (ti <= tj) {
        const size_t tile = static_cast<size_t>(ti) * p.T - static_cast<size_t>(ti) * (ti - 1) / 2 + (tj - ti);
        uint32_t e;
        const floatx4* src = part + tile * tile_f4 + slot_of(vi % BT, vj % BT, e);
        int s = 0;
        for (; s + 8 <= n; s += 8) {                                      // eight loads in flight, summed in order
          floatx4 w[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) w[k] = src[(s + k) * split_stride];
#pragma unroll
          for (int k = 0; k < 8; ++k) acc += w[k];
        }
        for (; s < n; ++s) acc += src[s * split_stride];
      } else {
        const size_t tile = static_cast<size_t>(tj) * p.T - static_cast<size_t>(tj) * (tj - 1) / 2 + (ti - tj);
        const float* base = reinterpret_cast<const float*>(part + tile * tile_f4);
        size_t off[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          uint32_t e;
          const uint32_t f4 = slot_of(vj % BT, (vi + k) % BT, e);
          off[k] = static_cast<size_t>(f4) * 4 + e;
        }
        int s = 0;
        for (; s + 2 <= n; s += 2) {
          const float* q0 = base + static_cast<size_t>(s) * split_stride * 4;
          const float* q1 = q0 + split_stride * 4;
          const float x0 = q0[off[0]], x1 = q0[off[1]], x2 = q0[off[2]], x3 = q0[off[3]];
          const float y0 = q1[off[0]], y1 = q1[off[1]], y2 = q1[off[2]], y3 = q1[off[3]];
          acc[0] += x0; acc[1] += x1; acc[2] += x2; acc[3] += x3;
          acc[0] += y0; acc[1] += y1; acc[2] += y2; acc[3] += y3;
        }
        for (; s < n; ++s) {
          const float* q = base + static_cast<size_t>(s) * split_stride * 4;
          acc[0] += q[off[0]]; acc[1] += q[off[1]]; acc[2] += q[off[2]]; acc[3] += q[off[3]];
        }
      }
      const uint32_t col = cgl * KK + tap_j;                              // result column inside the block
#pragma unroll
      for (int e = 0; e < 4; ++e) blk_lds[(e * KK + tap_i) * lw + col] = acc[e];
    }
  }
  __syncthreads();
  // the block, row by row: C[ci0 * KK + r][cj0 * KK + c]
  float* dst = p.C + static_cast<int64_t>(ci0) * KK * p.ldc + static_cast<int64_t>(cj0) * KK;
  for (uint32_t idx = tid; idx < rows * cols; idx += 256) {
    const uint32_t r = idx / cols, c = idx - r * cols;
    float v = p.alpha * blk_lds[r * lw + c];
    float* q = dst + static_cast<int64_t>(r) * p.ldc + c;
    if (p.beta != 0.f) v += p.beta * *q;
    *q = v;
    blk_lds[r * lw + c] = v;                                              // the mirror image stores the same value
  }
  if (grp_j == grp_i) return;
  __syncthreads();
  // the transposed block: C[cj0 * KK + c][ci0 * KK + r]
  float* dst_t = p.C + static_cast<int64_t>(cj0) * KK * p.ldc + static_cast<int64_t>(ci0) * KK;
  for (uint32_t idx = tid; idx < rows * cols; idx += 256) {
    const uint32_t c = idx / rows, r = idx - c * rows;
    dst_t[static_cast<int64_t>(c) * p.ldc + r] = blk_lds[r * lw + c];
  }
}

// The same for the gathered factors of a grouped launch: grid (column blocks x row blocks of the widest factor,
// factors with partial tiles); work groups beyond a narrower factor's blocks leave at once.
struct DtlGroupFinOut {
  int32_t factor, nparts, col_blocks, pad;
  int64_t first, ntiles;
};

template <int WR, int WC, int FR, int FC>
__global__ __launch_bounds__(256) void syrk_dtl_finalize_out_grouped_kernel(const DtlParams* __restrict__ factors,
                                                                            const DtlGroupFinOut* __restrict__ fins,
                                                                            const floatx4* __restrict__ ws) {
  const DtlGroupFinOut it = fins[blockIdx.y];
  const DtlParams p = factors[it.factor];
  const uint32_t row_block = blockIdx.x / it.col_blocks, col_block = blockIdx.x - row_block * it.col_blocks;
  dtl_finalize_out<WR, WC, FR, FC>(p, ws + it.first, it.ntiles, it.nparts, col_block, row_block);
}

// ---- host side ------------------------------------------------------------------------------------

constexpr int kDtlDirectSplits = 24;   // up to this many partials the epilogue pass sums them itself

struct DtlPlan {
  int bt;          // work-group tile: 64, 128, 192 or 256
  int T, nsplit;
  int group, ngroups;   // two-stage reduction: partials per first-stage sum, number of sums (0: single stage)
  int64_t ntiles, rows_per_split;
  size_t ws_bytes;
};

// 0: the built-in choice of the gather group / the cost model's tile size and split factor.  Only a tuning build
// (-DAK_TUNING_HOOKS) can pin them.
#ifdef AK_TUNING_HOOKS
static int g_force_group = 0;
static int g_force_bt = 0, g_force_ns = 0;
#else
constexpr int g_force_group = 0;
constexpr int g_force_bt = 0, g_force_ns = 0;
#endif

// Tile size and split-K factor from a small cost model (microseconds, constants measured on MI355X): the
// k-tiles of one split times the k-tile time of the most loaded CU, a fixed charge per work group, the
// partial-tile traffic and the reduction passes.
static DtlPlan dtl_plan_search(int64_t M, int64_t d, int64_t max_rows_per_split, bool gather) {
  struct Cand { int bt; int occ; double t_alone, t_shared, t_fix; };
  // t_alone: k-tile time of a work group that has its CU to itself, t_shared: with `occ` of them on the CU
  const Cand cands[4] = {{64, 4, 0.20, 0.20, 3.0},
                         {128, 2, gather ? 0.40 : 0.25, 0.59, 4.0},
                         {192, 1, gather ? 0.55 : 0.42, gather ? 0.55 : 0.42, 6.0},
                         {256, 1, gather ? 0.82 : 0.62, gather ? 0.82 : 0.62, 8.0}};
  const int64_t ktiles = (M + kDtlBK - 1) / kDtlBK;
  DtlPlan best{};
  double best_cost = 1e300;
  for (const Cand& c : cands) {
    if (g_force_bt != 0 && c.bt != g_force_bt) continue;
    if (g_force_bt == 0 && c.bt == 64 && d > 192) continue;
    if (g_force_bt == 0 && c.bt == 256 && d < 1024) continue;
    if (g_force_bt == 0 && c.bt == 192 && d < 384) continue;
    const int64_t T = (d + c.bt - 1) / c.bt, ntiles = T * (T + 1) / 2;
    const int64_t slots = 256 * c.occ;
    const int64_t ns_cap = ktiles / 4 < 1 ? 1 : (ktiles / 4 > 1024 ? 1024 : ktiles / 4);
    for (int64_t ns = 1; ns <= ns_cap; ++ns) {
      if (g_force_ns != 0 && ns != (g_force_ns < ns_cap ? g_force_ns : ns_cap)) continue;
      const int64_t kt_split = (ktiles + ns - 1) / ns;
      if (kt_split * kDtlBK > max_rows_per_split) continue;
      const int64_t ns_eff = (ktiles + kt_split - 1) / kt_split;
      const int64_t wgs = ntiles * ns_eff, rounds = (wgs + slots - 1) / slots;
      int64_t per_cu = (wgs + 255) / 256;
      if (per_cu > c.occ) per_cu = c.occ;
      const double t_kt = c.occ > 1 ? c.t_alone + (c.t_shared - c.t_alone) * (per_cu - 1) / (c.occ - 1) : c.t_alone;
      double cost = static_cast<double>(rounds) * (static_cast<double>(kt_split) * t_kt + c.t_fix);
      if (ns_eff > 1) {
        const double part_mb = static_cast<double>(wgs) * c.bt * c.bt * 4.0 * 1e-6;
        cost += 2.0 * part_mb / 5.0;                                // written once, read once, ~5 TB/s out of L2/MALL
        cost += ns_eff <= kDtlDirectSplits ? 3.0 + 0.08 * ns_eff : 7.0 + 0.3 * std::sqrt(static_cast<double>(ns_eff));
      }
      if (cost < best_cost) {
        best_cost = cost;
        best.bt = c.bt;
        best.T = static_cast<int>(T);
        best.ntiles = ntiles;
        best.rows_per_split = kt_split * kDtlBK;
      }
    }
  }
  if (best.bt == 0) {                                               // nothing fits the offset range
    best.bt = 128;
    best.T = static_cast<int>((d + 127) / 128);
    best.ntiles = static_cast<int64_t>(best.T) * (best.T + 1) / 2;
    best.rows_per_split = ((M + kDtlBK - 1) / kDtlBK) * kDtlBK;
  }
  best.nsplit = static_cast<int>((M + best.rows_per_split - 1) / best.rows_per_split);
  if (best.nsplit < 1) best.nsplit = 1;
  best.group = best.ngroups = 0;
  size_t parts = best.nsplit > 1 ? best.nsplit : 0;
  if (best.nsplit > kDtlDirectSplits) {
    best.group = static_cast<int>(std::ceil(std::sqrt(static_cast<double>(best.nsplit))));
    best.ngroups = (best.nsplit + best.group - 1) / best.group;
    parts += best.ngroups;
  }
  best.ws_bytes = parts * best.ntiles * best.bt * best.bt * sizeof(float);
  return best;
}

// The search above walks over up to 3 x 1024 candidates (tens of microseconds on the host): the same few shapes
// recur every step, so the plans are memoised.  Entry points may be called from several host threads.
static DtlPlan dtl_plan(int64_t M, int64_t d, int64_t max_rows_per_split, bool gather) {
  struct Key {
    int64_t M, d, rows;
    int gather, bt, ns;
    bool operator==(const Key& o) const {
      return M == o.M && d == o.d && rows == o.rows && gather == o.gather && bt == o.bt && ns == o.ns;
    }
  };
  struct Hash {
    size_t operator()(const Key& k) const {
      uint64_t h = 0x9e3779b97f4a7c15ull;
      for (uint64_t v : {static_cast<uint64_t>(k.M), static_cast<uint64_t>(k.d), static_cast<uint64_t>(k.rows),
                         static_cast<uint64_t>(k.gather), static_cast<uint64_t>(k.bt), static_cast<uint64_t>(k.ns)})
        h = (h ^ v) * 0xff51afd7ed558ccdull + (h >> 29);
      return static_cast<size_t>(h);
    }
  };
  static std::unordered_map<Key, DtlPlan, Hash> cache;
  static std::mutex lock;
  const Key key{M, d, max_rows_per_split, gather ? 1 : 0, g_force_bt, g_force_ns};
  std::lock_guard<std::mutex> guard(lock);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  if (cache.size() > 4096) cache.clear();
  const DtlPlan plan = dtl_plan_search(M, d, max_rows_per_split, gather);
  cache.emplace(key, plan);
  return plan;
}

// Channels per column block of the LDS-staged reduction pass of a gathered factor (0: use the pass by output
// position): a divisor of G small enough for 64 KB of LDS and for at least ~2 work groups per CU.
static int dtl_blk_channels(const DtlParams& p) {
  if (p.KK < 2 || p.Cin % 4 != 0 || p.G % 4 != 0 || p.Cin % p.G != 0) return 0;
  int cpb = 0;
  for (int c = p.G; c >= 4; c /= 2) {
    if (p.G % c != 0) break;
    const size_t lds = static_cast<size_t>(4 * p.KK) * (c * p.KK + 1) * sizeof(float);
    if (lds > 64 * 1024) continue;
    cpb = c;
    const int64_t wgs = static_cast<int64_t>(p.Cin / c) * (p.Cin / 4) / 2;     // about half are above the diagonal
    if (wgs >= 512) break;
  }
  return cpb;
}

template <int WR, int WC, int FR, int FC, bool GATHER>
static int dtl_launch_cfg(const DtlParams& p, const DtlPlan& pl, hipStream_t stream) {
  using Cfg = DtlCfg<WR, WC, FR, FC, GATHER>;
  auto kern = syrk_dtl_kernel<WR, WC, FR, FC, GATHER>;
  if (Cfg::LDS_BYTES > 64 * 1024) {
    static bool attr_set = false;     // idempotent; a race sets it twice at worst
    if (!attr_set) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              Cfg::LDS_BYTES) != hipSuccess)
        return AK_ERR_LAUNCH;
      attr_set = true;
    }
  }
  const unsigned ntiles = static_cast<unsigned>(pl.ntiles);
  hipLaunchKernelGGL(kern, dim3(ntiles, static_cast<unsigned>(p.nsplit)), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, stream, p);
  if (p.nsplit > 1) {
    const size_t tile_f4 = static_cast<size_t>(Cfg::BT) * Cfg::BT / 4;
    const floatx4* part = reinterpret_cast<const floatx4*>(p.ws);
    int n = p.nsplit;
    if (pl.ngroups > 0) {
      floatx4* sums = reinterpret_cast<floatx4*>(p.ws) + static_cast<size_t>(p.nsplit) * pl.ntiles * tile_f4;
      hipLaunchKernelGGL((syrk_dtl_reduce_kernel<Cfg::NW * 64>), dim3(ntiles, 4 * FR * FC, pl.ngroups),
                         dim3(Cfg::NW * 64), 0, stream, part, sums, p.nsplit, pl.group, tile_f4);
      part = sums;
      n = pl.ngroups;
    }
    if constexpr (GATHER) {
      const unsigned d = static_cast<unsigned>(p.d);
      const int cpb = dtl_blk_channels(p);
      if (cpb > 0) {
        const size_t lds = static_cast<size_t>(4 * p.KK) * (cpb * p.KK + 1) * sizeof(float);
        hipLaunchKernelGGL((syrk_dtl_finalize_blk_kernel<WR, WC, FR, FC>), dim3(p.Cin / cpb, p.Cin / 4), dim3(256), lds,
                           stream, p, part, pl.ntiles, n, cpb);
      } else {
        hipLaunchKernelGGL((syrk_dtl_finalize_out_kernel<WR, WC, FR, FC>), dim3((d + 63) / 64, (d + 15) / 16),
                           dim3(256), 0, stream, p, part, pl.ntiles, n);
      }
    } else {
      hipLaunchKernelGGL((syrk_dtl_finalize_kernel<WR, WC, FR, FC, GATHER>), dim3(ntiles, 4 * FR * FC),
                         dim3(Cfg::NW * 64), 0, stream, p, part, n);
    }
  }
  return check_launch();
}

template <bool GATHER>
static int dtl_launch(DtlParams& p, const DtlPlan& pl, void* ws, size_t ws_bytes, hipStream_t stream) {
  if (pl.ws_bytes > 0 && (ws == nullptr || ws_bytes < pl.ws_bytes)) return AK_ERR_WORKSPACE;
  p.T = pl.T;
  p.nsplit = pl.nsplit;
  p.rows_per_split = pl.rows_per_split;
  p.ws = static_cast<float*>(ws);
  if (pl.bt == 64) return dtl_launch_cfg<2, 2, 1, 1, GATHER>(p, pl, stream);
  if (pl.bt == 256) return dtl_launch_cfg<2, 4, 4, 2, GATHER>(p, pl, stream);
  if (pl.bt == 192) return dtl_launch_cfg<2, 2, 3, 3, GATHER>(p, pl, stream);
  return dtl_launch_cfg<2, 2, 2, 2, GATHER>(p, pl, stream);
}

bool syrk_dtl_plain_ok(const void* X, int64_t M, int64_t d, int64_t ldx) {
  return M > 0 && d % 8 == 0 && ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(X) & 15) == 0 &&
         ldx * 2 * static_cast<int64_t>(kDtlBK) <= static_cast<int64_t>(kDtlRange);
}

static int64_t plain_max_rows(int64_t ldx) { return static_cast<int64_t>(kDtlRange) / (ldx * 2); }

size_t syrk_dtl_plain_ws_bytes(int64_t M, int64_t d, int64_t ldx) {
  return dtl_plan(M, d, plain_max_rows(ldx), false).ws_bytes;
}

int syrk_dtl_plain(const void* X, int64_t M, int64_t d, int64_t ldx, float alpha, float beta, float* C,
                   int64_t ldc, void* ws, size_t ws_bytes, hipStream_t stream) {
  DtlParams p{};
  p.X = X; p.C = C; p.M = M; p.d = d; p.ldc = ldc;
  p.row_bytes = static_cast<uint32_t>(ldx * 2);
  p.alpha = alpha; p.beta = beta;
  p.Cin = 1; p.KK = 1;
  const DtlPlan pl = dtl_plan(M, d, plain_max_rows(ldx), false);
  if (pl.rows_per_split > plain_max_rows(ldx)) return AK_ERR_UNSUPPORTED;
  return dtl_launch<false>(p, pl, ws, ws_bytes, stream);
}

static bool nhwc_ok(const void* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw,
                    int ph, int pw, int64_t& Ho, int64_t& Wo) {
  if (x == nullptr || N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 || ph < 0 ||
      pw < 0)
    return false;
  Ho = (H + 2 * ph - kh) / sh + 1;
  Wo = (W + 2 * pw - kw) / sw + 1;
  if (Ho <= 0 || Wo <= 0) return false;
  return true;
}

// Gather geometry of a channels-last convolution input; false when the direct-to-LDS kernel cannot read it (16-byte
// chunks must not straddle taps, offsets must fit the 32-bit buffer range, and the magic divisions by Wo, Ho, C and
// kw must be exact over their operand ranges).
static bool dtl_gather_params(DtlParams& p, const void* x, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw,
                              int sh, int sw, int ph, int pw, int64_t Ho, int64_t Wo) {
  const int64_t d = C * kh * kw, M = N * Ho * Wo;
  if (C % 8 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0) return false;
  if (N * H * W * C * 2 > static_cast<int64_t>(kDtlRange)) return false;
  if (M * (Wo > Ho ? Wo : Ho) >= (1ll << 32) || (d + 256) * d >= (1ll << 32)) return false;
  p.X = x; p.M = M; p.d = d;
  p.Cin = static_cast<int>(C); p.H = static_cast<int>(H); p.W = static_cast<int>(W);
  p.kw = kw; p.KK = kh * kw; p.sh = sh; p.sw = sw; p.ph = ph; p.pw = pw;
  p.Ho = static_cast<int>(Ho); p.Wo = static_cast<int>(Wo);
  p.mWo = make_magic(p.Wo); p.mHo = make_magic(p.Ho); p.mKw = make_magic(kw);
  p.G = g_force_group > 0 && p.Cin % g_force_group == 0 ? g_force_group : (d >= 3456 ? 8 : (p.Cin % 32 == 0 ? 32 : p.Cin));
  p.mBlk = make_magic(p.G * p.KK); p.mG = make_magic(p.G); p.mKK = make_magic(p.KK);
  return true;
}

// ---- many factors in one launch ---------------------------------------------------------------------------------
// The factors of a whole forward or backward pass are small launches when taken one by one: a few tiles, split
// along the rows to fill the device, each paying its ramp, its tail, its partial tiles and a reduction launch.
// Taken together they fill the device with long work items: one launch per tile class, few splits, one reduction
// launch per class.  A factor is described by kGroupSpecInts int64:
//   [0] kind (0: X^T X of a bf16 [M, d] matrix, 1: unfolded channels-last bf16 [N, C, H, W] input)
//   [1] operand address  [2] result address (fp32 [d, d])  [3] ldc  [4] alpha bits | beta bits << 32
//   kind 0: [5] M  [6] d  [7] ldx          kind 1: [5] N  [6] C  [7] H  [8] W  [9] kh  [10] kw  [11..14] sh sw ph pw
constexpr int kGroupSpecInts = 16;
constexpr int kGroupClasses = 4;           // plain 128 / 192, gathered 128 / 192
constexpr int kGroupMaxSplits = 96;         // partial tiles per tile that the reduction pass sums, one after the other

struct GroupFactor {
  DtlParams p;
  int cls, bt;
  int64_t ktiles, ntiles, kt_split, part_base;   // part_base: float4 index of this factor's partial tiles
  int nsplit;
};

static int group_class(bool gather, int64_t d, int& bt) {
  if (!gather) { bt = d >= 1536 ? 192 : 128; return bt == 128 ? 0 : 1; }
  bt = d >= 576 ? 192 : 128;
  return bt == 128 ? 2 : 3;
}

static bool group_decode(const int64_t* r, GroupFactor& f, int64_t& max_rows_per_split) {
  DtlParams& p = f.p;
  p = DtlParams{};
  const void* x = reinterpret_cast<const void*>(r[1]);
  p.C = reinterpret_cast<float*>(r[2]);
  p.ldc = r[3];
  const uint32_t abits = static_cast<uint32_t>(r[4] & 0xffffffffll), bbits = static_cast<uint32_t>(r[4] >> 32);
  std::memcpy(&p.alpha, &abits, 4);
  std::memcpy(&p.beta, &bbits, 4);
  if (x == nullptr || p.C == nullptr) return false;
  bool gather;
  if (r[0] == 0) {
    const int64_t M = r[5], d = r[6], ldx = r[7];
    if (M <= 0 || d <= 0 || ldx < d || p.ldc < d || !syrk_dtl_plain_ok(x, M, d, ldx)) return false;
    p.X = x; p.M = M; p.d = d;
    p.row_bytes = static_cast<uint32_t>(ldx * 2);
    p.Cin = 1; p.KK = 1;
    max_rows_per_split = plain_max_rows(ldx);
    gather = false;
  } else if (r[0] == 1) {
    const int64_t N = r[5], C = r[6], H = r[7], W = r[8];
    const int kh = static_cast<int>(r[9]), kw = static_cast<int>(r[10]), sh = static_cast<int>(r[11]),
              sw = static_cast<int>(r[12]), ph = static_cast<int>(r[13]), pw = static_cast<int>(r[14]);
    int64_t Ho, Wo;
    if (!nhwc_ok(x, N, C, H, W, kh, kw, sh, sw, ph, pw, Ho, Wo)) return false;
    if (conv_patch_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw) > 0) return false;     // the window kernel's case
    if (conv_corr_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw) > 0) return false;      // the shifted-correlation form's
    if (p.ldc < C * kh * kw) return false;
    if (!dtl_gather_params(p, x, N, C, H, W, kh, kw, sh, sw, ph, pw, Ho, Wo)) return false;
    // the widest factors fill the device on their own, with the 256-wide tile of 8 waves, whose register budget
    // has no room for a descriptor read from memory
    if (p.d >= 3456) return false;
    max_rows_per_split = INT64_MAX;
    gather = true;
  } else {
    return false;
  }
  if (!syrk_beta_ok(p.beta, p.d, p.ldc)) return false;
  f.cls = group_class(gather, p.d, f.bt);
  p.T = static_cast<int>((p.d + f.bt - 1) / f.bt);
  f.ntiles = static_cast<int64_t>(p.T) * (p.T + 1) / 2;
  f.ktiles = (p.M + kDtlBK - 1) / kDtlBK;
  return true;
}

struct GroupPlan {
  std::vector<GroupFactor> factors;
  std::vector<DtlGroupItem> items[kGroupClasses];
  std::vector<DtlGroupFin> fins[kGroupClasses];           // plain classes: reduction by accumulator slot
  std::vector<DtlGroupFinOut> fins_out[kGroupClasses];    // gathered classes: reduction by output position
  unsigned fin_out_blocks[kGroupClasses] = {};
  size_t ws_f4 = 0;                       // partial tiles, in float4
  size_t off_factors = 0, off_items[kGroupClasses], off_fins[kGroupClasses], off_fins_out[kGroupClasses], table_bytes = 0;
};

static int group_plan(const int64_t* specs, int n, GroupPlan& g) {
  if (specs == nullptr || n <= 0) return AK_ERR_ARG;
  g.factors.resize(n);
  std::vector<int64_t> max_rows(n);
  int64_t work[kGroupClasses] = {0, 0, 0, 0};
  for (int i = 0; i < n; ++i) {
    if (!group_decode(specs + static_cast<size_t>(i) * kGroupSpecInts, g.factors[i], max_rows[i])) return AK_ERR_UNSUPPORTED;
    for (int j = 0; j < i; ++j)           // two items writing one result would race
      if (g.factors[j].p.C == g.factors[i].p.C) return AK_ERR_ARG;
    work[g.factors[i].cls] += g.factors[i].ntiles * g.factors[i].ktiles;
  }
  size_t ws_f4 = 0;
  for (int c = 0; c < kGroupClasses; ++c) {
    if (work[c] == 0) continue;
    const int bt = (c == 0 || c == 2) ? 128 : 192;
    const int64_t slots = 256 * (bt == 128 ? 2 : 1);
    // The longest item a factor may have, in k-tiles ("chunk"): longer row ranges are split.  Candidates: no split at
    // all, and 1/4 or 1/8 of the work per slot (coarser items balance well on paper only: work groups do not all
    // run at one speed); each is judged by the finishing time of a greedy assignment of its items, longest first,
    // to the slots (what the dispatcher does with the work groups in launch order) plus the traffic of the partial
    // tiles it causes.  A group of a few wide factors thus stays unsplit, a pass of many narrow ones gets a few
    // splits each.
    auto splits_of = [&](int i, int64_t chunk) {
      const GroupFactor& f = g.factors[i];
      int64_t ns = (f.ktiles + chunk - 1) / chunk;
      if (ns > kGroupMaxSplits) ns = kGroupMaxSplits;
      const int64_t max_kt = max_rows[i] / kDtlBK;
      if ((f.ktiles + ns - 1) / ns > max_kt) ns = (f.ktiles + max_kt - 1) / max_kt;
      return ns < 1 ? int64_t{1} : ns;
    };
    int64_t longest = 0;
    for (int i = 0; i < n; ++i) {
      if (g.factors[i].cls != c) continue;
      if (max_rows[i] / kDtlBK < 1) return AK_ERR_UNSUPPORTED;
      longest = std::max(longest, g.factors[i].ktiles);
    }
    // microseconds per k-tile of a work group: two 128-wide ones share a CU (dtl_plan_search's t_shared), a 192-wide
    // one has it to itself
    const double t_kt = bt == 128 ? 0.55 : 0.45;
    int64_t chunk = longest;
    double best_cost = 1e300;
    for (int k = 0; k <= 4; k += (k == 0 ? 3 : 1)) {
      int64_t cand = k == 0 ? longest : (work[c] + slots * (1 << (k - 1)) - 1) / (slots * (1 << (k - 1)));
      if (cand < 32) cand = 32;
      if (cand > longest) cand = longest;
      std::vector<int64_t> lens;                            // item lengths, longest first
      double part_mb = 0.0;
      int64_t most_splits = 1;
      for (int i = 0; i < n; ++i) {
        const GroupFactor& f = g.factors[i];
        if (f.cls != c) continue;
        const int64_t ns = splits_of(i, cand), len = (f.ktiles + ns - 1) / ns;
        lens.insert(lens.end(), static_cast<size_t>(ns * f.ntiles), len);
        if (ns > 1) part_mb += static_cast<double>(ns * f.ntiles) * bt * bt * 4.0 * 1e-6;
        most_splits = std::max(most_splits, ns);
      }
      std::sort(lens.begin(), lens.end(), std::greater<int64_t>());
      std::priority_queue<int64_t, std::vector<int64_t>, std::greater<int64_t>> busy;   // finishing times of the slots
      int64_t makespan = 0;
      for (int64_t len : lens) {
        int64_t start = 0;
        if (static_cast<int64_t>(busy.size()) >= slots) { start = busy.top(); busy.pop(); }
        busy.push(start + len);
        makespan = std::max(makespan, start + len);
      }
      // partial tiles: written once, read once, ~5 TB/s out of L2 / MALL; the reduction pass: a launch and a chain
      // of dependent reads as long as the largest split count
      const double cost = static_cast<double>(makespan) * t_kt + 2.0 * part_mb / 5.0 +
                          (part_mb > 0 ? 4.0 + 0.15 * static_cast<double>(most_splits) : 0.0);
      if (cost < best_cost) { best_cost = cost; chunk = cand; }
    }
    std::vector<int> order;
    for (int i = 0; i < n; ++i) {
      GroupFactor& f = g.factors[i];
      if (f.cls != c) continue;
      const int64_t ns = splits_of(i, chunk);
      f.kt_split = (f.ktiles + ns - 1) / ns;
      f.nsplit = static_cast<int>((f.ktiles + f.kt_split - 1) / f.kt_split);
      f.p.nsplit = f.nsplit;
      f.p.rows_per_split = f.kt_split * kDtlBK;
      f.part_base = -1;
      if (f.nsplit > 1) {
        f.part_base = static_cast<int64_t>(ws_f4);
        ws_f4 += static_cast<size_t>(f.nsplit) * f.ntiles * (static_cast<size_t>(bt) * bt / 4);
      }
      order.push_back(i);
    }
    // the longest items first: the short ones fill the tail
    std::stable_sort(order.begin(), order.end(),
                     [&](int a, int b) { return g.factors[a].kt_split > g.factors[b].kt_split; });
    const int64_t tile_f4 = static_cast<int64_t>(bt) * bt / 4;
    for (int i : order) {
      const GroupFactor& f = g.factors[i];
      for (int s = 0; s < f.nsplit; ++s)
        for (int64_t t = 0; t < f.ntiles; ++t) {
          DtlGroupItem it;
          it.factor = i;
          it.tile = static_cast<int32_t>(t);
          it.k_begin_tile = static_cast<int32_t>(s * f.kt_split);
          it.k_tiles = static_cast<int32_t>(f.kt_split);
          it.partial = f.nsplit > 1 ? f.part_base + (static_cast<int64_t>(s) * f.ntiles + t) * tile_f4 : -1;
          g.items[c].push_back(it);
        }
      if (f.nsplit > 1 && c >= 2) {
        DtlGroupFinOut fin;
        const unsigned d = static_cast<unsigned>(f.p.d);
        fin.factor = i;
        fin.nparts = f.nsplit;
        fin.col_blocks = static_cast<int32_t>((d + 63) / 64);
        fin.pad = 0;
        fin.first = f.part_base;
        fin.ntiles = f.ntiles;
        g.fins_out[c].push_back(fin);
        g.fin_out_blocks[c] = std::max(g.fin_out_blocks[c], ((d + 63) / 64) * ((d + 15) / 16));
      }
      if (f.nsplit > 1 && c < 2)
        for (int64_t t = 0; t < f.ntiles; ++t) {
          DtlGroupFin fin;
          fin.factor = i;
          fin.tile = static_cast<int32_t>(t);
          fin.nparts = f.nsplit;
          fin.pad = 0;
          fin.first = f.part_base + t * tile_f4;
          fin.stride = f.ntiles * tile_f4;
          g.fins[c].push_back(fin);
        }
    }
  }
  g.ws_f4 = ws_f4;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off += (bytes + 255) & ~static_cast<size_t>(255); return at; };
  g.off_factors = take(sizeof(DtlParams) * n);
  for (int c = 0; c < kGroupClasses; ++c) {
    g.off_items[c] = take(sizeof(DtlGroupItem) * g.items[c].size());
    g.off_fins[c] = take(sizeof(DtlGroupFin) * g.fins[c].size());
    g.off_fins_out[c] = take(sizeof(DtlGroupFinOut) * g.fins_out[c].size());
  }
  g.table_bytes = off;
  return AK_OK;
}

template <int WR, int WC, int FR, int FC, bool GATHER>
static int group_launch_class(const GroupPlan& g, int c, const unsigned char* tables, floatx4* ws, hipStream_t stream) {
  using Cfg = DtlCfg<WR, WC, FR, FC, GATHER>;
  if (g.items[c].empty()) return AK_OK;
  auto kern = syrk_dtl_grouped_kernel<WR, WC, FR, FC, GATHER>;
  if (Cfg::LDS_BYTES > 64 * 1024) {
    static bool attr_set = false;     // idempotent; a race sets it twice at worst
    if (!attr_set) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              Cfg::LDS_BYTES) != hipSuccess)
        return AK_ERR_LAUNCH;
      attr_set = true;
    }
  }
  const DtlParams* factors = reinterpret_cast<const DtlParams*>(tables + g.off_factors);
  const DtlGroupItem* items = reinterpret_cast<const DtlGroupItem*>(tables + g.off_items[c]);
  hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(g.items[c].size())), dim3(Cfg::NW * 64), Cfg::LDS_BYTES, stream,
                     factors, items, ws);
  if (!g.fins[c].empty()) {
    const DtlGroupFin* fins = reinterpret_cast<const DtlGroupFin*>(tables + g.off_fins[c]);
    hipLaunchKernelGGL((syrk_dtl_finalize_grouped_kernel<WR, WC, FR, FC, GATHER>),
                       dim3(static_cast<unsigned>(g.fins[c].size()), 4 * FR * FC), dim3(Cfg::NW * 64), 0, stream, factors,
                       fins, static_cast<const floatx4*>(ws));
  }
  if constexpr (GATHER) {
    if (!g.fins_out[c].empty()) {
      const DtlGroupFinOut* fins = reinterpret_cast<const DtlGroupFinOut*>(tables + g.off_fins_out[c]);
      hipLaunchKernelGGL((syrk_dtl_finalize_out_grouped_kernel<WR, WC, FR, FC>),
                         dim3(g.fin_out_blocks[c], static_cast<unsigned>(g.fins_out[c].size())), dim3(256), 0, stream,
                         factors, fins, static_cast<const floatx4*>(ws));
    }
  }
  return check_launch();
}

}  // namespace ak

extern "C" int ak_syrk_group_eligible(const int64_t* spec) {
  if (spec == nullptr) return 0;
  ak::GroupFactor f;
  int64_t max_rows;
  return ak::group_decode(spec, f, max_rows) && max_rows >= ak::kDtlBK ? 1 : 0;
}

extern "C" int ak_syrk_group_sizes(const int64_t* specs, int n, size_t* table_bytes, size_t* ws_bytes) {
  if (table_bytes == nullptr || ws_bytes == nullptr) return AK_ERR_ARG;
  ak::GroupPlan g;
  const int rc = ak::group_plan(specs, n, g);
  if (rc != AK_OK) return rc;
  *table_bytes = g.table_bytes;
  *ws_bytes = g.ws_f4 * sizeof(ak::floatx4);
  return AK_OK;
}

extern "C" int ak_syrk_group_launch(const int64_t* specs, int n, void* host_stage, void* dev_tables, size_t table_bytes,
                                    void* ws, size_t ws_bytes, ak_stream_t stream) {
  ak::GroupPlan g;
  int rc = ak::group_plan(specs, n, g);
  if (rc != AK_OK) return rc;
  if (host_stage == nullptr || dev_tables == nullptr || table_bytes < g.table_bytes) return AK_ERR_WORKSPACE;
  if (g.ws_f4 > 0 && (ws == nullptr || ws_bytes < g.ws_f4 * sizeof(ak::floatx4))) return AK_ERR_WORKSPACE;
  unsigned char* h = static_cast<unsigned char*>(host_stage);
  ak::DtlParams* hf = reinterpret_cast<ak::DtlParams*>(h + g.off_factors);
  for (int i = 0; i < n; ++i) hf[i] = g.factors[i].p;
  for (int c = 0; c < ak::kGroupClasses; ++c) {
    if (!g.items[c].empty())
      std::memcpy(h + g.off_items[c], g.items[c].data(), sizeof(ak::DtlGroupItem) * g.items[c].size());
    if (!g.fins[c].empty())
      std::memcpy(h + g.off_fins[c], g.fins[c].data(), sizeof(ak::DtlGroupFin) * g.fins[c].size());
    if (!g.fins_out[c].empty())
      std::memcpy(h + g.off_fins_out[c], g.fins_out[c].data(), sizeof(ak::DtlGroupFinOut) * g.fins_out[c].size());
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (hipMemcpyAsync(dev_tables, host_stage, g.table_bytes, hipMemcpyHostToDevice, s) != hipSuccess) return AK_ERR_LAUNCH;
  const unsigned char* t = static_cast<const unsigned char*>(dev_tables);
  ak::floatx4* w = static_cast<ak::floatx4*>(ws);
  if ((rc = ak::group_launch_class<2, 2, 2, 2, false>(g, 0, t, w, s)) != AK_OK) return rc;
  if ((rc = ak::group_launch_class<2, 2, 3, 3, false>(g, 1, t, w, s)) != AK_OK) return rc;
  if ((rc = ak::group_launch_class<2, 2, 2, 2, true>(g, 2, t, w, s)) != AK_OK) return rc;
  return ak::group_launch_class<2, 2, 3, 3, true>(g, 3, t, w, s);
}

#ifdef AK_TUNING_HOOKS
// Tuning builds only: pins the channel group size of the gathered column order (0: built-in choice).
extern "C" void ak_debug_force_gather_group(int group) { ak::g_force_group = group; }

// Tuning builds only: pins the tile size (64/128/256) and split-K factor of the direct-to-LDS SYRK; (0, 0) restores
// the cost model.
extern "C" void ak_debug_force_syrk_plan(int bt, int nsplit) {
  ak::g_force_bt = bt;
  ak::g_force_ns = nsplit;
}
#endif

extern "C" size_t ak_conv_syrk_nhwc_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                                             int sw, int ph, int pw) {
  int64_t Ho, Wo;
  if (!ak::nhwc_ok(reinterpret_cast<const void*>(16), N, C, H, W, kh, kw, sh, sw, ph, pw, Ho, Wo)) return 0;
  const size_t patch = ak::conv_patch_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw);
  if (patch > 0) return patch;
  const size_t corr = ak::conv_corr_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw);
  return std::max(corr, ak::dtl_plan(N * Ho * Wo, C * kh * kw, INT64_MAX, true).ws_bytes);
}

extern "C" int ak_conv_syrk_nhwc(const void* x, int dtype, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw,
                                 int sh, int sw, int ph, int pw, float alpha, float beta, float* A, int64_t lda,
                                 void* ws, size_t ws_bytes, ak_stream_t stream) {
  int64_t Ho, Wo;
  if (A == nullptr || !ak::nhwc_ok(x, N, C, H, W, kh, kw, sh, sw, ph, pw, Ho, Wo)) return AK_ERR_ARG;
  const int64_t d = C * kh * kw, M = N * Ho * Wo;
  if (lda < d) return AK_ERR_ARG;
  if (dtype != AK_BF16 && dtype != AK_F32 && dtype != AK_F32_AS_BF16) return AK_ERR_ARG;
  if (!ak::syrk_beta_ok(beta, d, lda)) return AK_ERR_UNSUPPORTED;
  {  // few input channels: the window kernel, any dtype and channel count
    const int rc = ak::conv_patch_syrk(x, dtype, H * W * C, 1, W * C, C, N, C, H, W, kh, kw, sh, sw, ph, pw, alpha, beta,
                                       A, lda, ws, ws_bytes, static_cast<hipStream_t>(stream));
    if (rc != AK_ERR_UNSUPPORTED) return rc;
  }
  if (dtype != AK_BF16) return AK_ERR_UNSUPPORTED;
  {  // 3 x 3, stride 1, padding 1: shifted correlations instead of the unfolded input
    const int rc = ak::conv_corr_syrk(x, N, C, H, W, kh, kw, sh, sw, ph, pw, alpha, beta, A, lda, ws, ws_bytes,
                                      static_cast<hipStream_t>(stream));
    if (rc != AK_ERR_UNSUPPORTED) return rc;
  }
  ak::DtlParams p{};
  if (!ak::dtl_gather_params(p, x, N, C, H, W, kh, kw, sh, sw, ph, pw, Ho, Wo)) return AK_ERR_UNSUPPORTED;
  p.C = A; p.ldc = lda;
  p.alpha = alpha; p.beta = beta;
  const ak::DtlPlan pl = ak::dtl_plan(M, d, INT64_MAX, true);
  return ak::dtl_launch<true>(p, pl, ws, ws_bytes, static_cast<hipStream_t>(stream));
}
