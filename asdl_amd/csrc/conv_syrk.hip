// A <- beta*A + alpha * sum over output positions of patch patch^T, with the im2col unfold
// fused: the patch matrix [n, c*kh*kw, h_out*w_out] never exists in memory.
//
// Row index of A: i = (c, ky, kx).  Contraction index: k = (n, oy, ox).  Consecutive ox are
// consecutive in NCHW memory, so the contraction index is the contiguous one and an MFMA
// operand (8 consecutive k for one i) is 16 contiguous bytes -- provided it is 16-byte
// aligned in LDS.  The kernel therefore stages, per panel of 64*TI rows of A and per block of
// R x WC output positions, one LDS row for every (channel, kx, input row):
//     plane[c][kx][r][q] = x[n, c, oy0*sh - ph + r, (ox0 + q)*sw + kx - pw]   (0 outside)
// i.e. the kx shift (and the sw decimation) is applied on the way in, with unaligned 16-byte
// global loads (row edges are masked, not gathered), and every MFMA fragment afterwards is one
// aligned ds_read_b128 at
//     base(i) + (oy_local*sh)*RS + 8*u,   base(i) = c_local*CS + kx*PS + ky*RS.
// The ky shift is a whole-row offset and costs nothing.  RS, PS, CS carry padding chosen on the
// host so that 8 consecutive rows i hit 8 different 16-byte bank groups.  The k-space is padded
// to a multiple of 8 per output row with zeros.  Global loads of stage s+1 are issued into
// registers before the MFMAs of stage s; LDS fragments of k-step t+1 are read before the MFMAs of
// k-step t.  kh = kw = 1 with H = 1 is the plain "X X^T, contraction contiguous" case used for
// Conv2d.cov_kron_B and for Shampoo's G G^T.
#include "common.hpp"
#include <map>
#include <mutex>
#include <utility>

namespace ak {

constexpr int CH = 8;   // 16-byte chunks one thread may stage per panel and stage (register prefetch depth)

struct ConvSyrkParams {
  const void* x;
  int64_t N, C, H, W;
  int kh, kw, sh, sw, ph, pw, Ho, Wo;
  int64_t d;
  float alpha, beta;
  float* A;
  int64_t lda;
  float* ws;
  int T, nsplit;
  int KK;        // kh*kw
  int R;         // output rows per stage
  int WC;        // output columns per stage (multiple of 8)
  int U;         // WC / 8 k-units per output row
  int RI;        // input rows per stage = (R-1)*sh + kh
  int RS, PS, CS;   // LDS strides in elements: input row, kx plane, channel
  int NCmax;     // channels a panel can touch
  int panel_elems;
  int RB, CB;    // row blocks per image, column chunks per row
  int64_t total_stages, stages_per_split;
  int64_t total_elems;    // N*C*H*W
  uint32_t mKK, mKw, mRI, mKwRI, mCPR, mCB, mRBCB;   // magic multipliers for division
  int RP, dcl, dkx, dr;   // LDS rows staged per pass of the work group, and that step decomposed as (channel, kx, row)
};


typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 __attribute__((aligned(2))) uint4_a2;
typedef u32x4 __attribute__((aligned(4))) uint4_a4;

template <typename T> struct Elem;
template <> struct Elem<uint16_t> { static constexpr int E = 8; typedef uint4_a2 vec_u; };
template <> struct Elem<float> { static constexpr int E = 4; typedef uint4_a4 vec_u; };

#define AK_LDS __attribute__((address_space(3)))

// What one thread stages for one panel: chunk m = tid % CPR of LDS rows row0, row0 + RP, ... (at most CH).
// The (channel, kx, input row) of every such row is the same in every stage, so it is decoded once.
struct ChunkTab {
  int goff[CH];   // ((c_lo + cl) * H + r) * W : element offset of the input row for oy0*sh - ph == 0
  int pk[CH];     // r | kx << 8 | (LDS byte offset / 16) << 12 ; r = 0xff marks an unused slot
};

__device__ __forceinline__ void build_tab(ChunkTab& tab, const ConvSyrkParams& p, int c_lo, int nc, int row0, int q0,
                                          int E) {
  const int kwRI = p.kw * p.RI;
  const int total_rows = nc * kwRI;
  int cl = static_cast<int>(fastdiv(row0, p.mKwRI, kwRI));
  const int t2 = row0 - cl * kwRI;
  int kx = static_cast<int>(fastdiv(t2, p.mRI, p.RI));
  int r = t2 - kx * p.RI;
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const bool used = row0 < p.RP && row0 + u * p.RP < total_rows;
    const int loff = cl * p.CS + kx * p.PS + r * p.RS + q0;
    tab.goff[u] = used ? ((c_lo + cl) * static_cast<int>(p.H) + r) * static_cast<int>(p.W) : 0;
    tab.pk[u] = used ? (r | (kx << 8) | ((loff / E) << 12)) : 0xff;
    r += p.dr; kx += p.dkx; cl += p.dcl;
    if (r >= p.RI) { r -= p.RI; kx += 1; }
    if (kx >= p.kw) { kx -= p.kw; cl += 1; }
  }
}

struct StageGeom {
  int64_t img;     // element offset of image n plus (oy0*sh - ph) * W
  int iy0, xq, W_eff, RI_eff;
};

// Issues this thread's global loads of one panel for one stage into registers (no LDS traffic).
template <typename T>
__device__ __forceinline__ void fetch_panel(u32x4 (&reg)[CH], const ChunkTab& tab, const ConvSyrkParams& p,
                                            const T* __restrict__ x, const StageGeom& sg, int q0, int nch) {
  constexpr int E = Elem<T>::E;
  const int xq = sg.xq + q0 * p.sw;
  const int q_room = sg.W_eff - q0;          // valid output columns from q0 on
  const int span = (p.sw == 1) ? E : 2 * E;  // elements touched by the vector path
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (u < nch) {
      const int r = tab.pk[u] & 0xff, kx = (tab.pk[u] >> 8) & 0xf;
      const int iy = sg.iy0 + r, x0 = xq + kx;
      if (q_room > 0 && r < sg.RI_eff && static_cast<unsigned>(iy) < static_cast<unsigned>(p.H)) {
        const int64_t row_off = sg.img + tab.goff[u];
        const T* src = x + row_off;
        // valid elements of this chunk: e in [e_lo, e_hi)
        int e_lo, lim_w;                                        // lim_w: first e with x0 + e*sw >= W
        if (p.sw == 1) { e_lo = max(-x0, 0); lim_w = static_cast<int>(p.W) - x0; }
        else if (p.sw == 2) { e_lo = max((1 - x0) >> 1, 0); lim_w = (static_cast<int>(p.W) - x0 + 1) >> 1; }
        else { e_lo = x0 < 0 ? (-x0 + p.sw - 1) / p.sw : 0; lim_w = (static_cast<int>(p.W) - x0 + p.sw - 1) / p.sw; }
        const int e_hi = min(E, min(lim_w, q_room));
        if (p.sw <= 2 && row_off + x0 >= 0 && row_off + x0 + span <= p.total_elems) {
          // the 16 (32) bytes lie inside the tensor: load them whole and zero what falls outside the row
          u32x4 w;
          if (p.sw == 1) {
            w = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0);
          } else {
            const u32x4 lo = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0);
            const u32x4 hi = *reinterpret_cast<const typename Elem<T>::vec_u*>(src + x0 + E);
            if constexpr (sizeof(T) == 2) {
              w.x = (lo.x & 0xffffu) | (lo.y << 16);
              w.y = (lo.z & 0xffffu) | (lo.w << 16);
              w.z = (hi.x & 0xffffu) | (hi.y << 16);
              w.w = (hi.z & 0xffffu) | (hi.w << 16);
            } else {
              w.x = lo.x; w.y = lo.z; w.z = hi.x; w.w = hi.z;
            }
          }
          if (e_lo > 0 || e_hi < E) {
            uint32_t d4[4] = {w.x, w.y, w.z, w.w};
            if constexpr (sizeof(T) == 2) {
              // bit e of `keep` set <=> element e valid; expand pairs of bits to 16-bit lane masks
              const uint32_t keep = ((1u << max(e_hi, 0)) - 1u) & ~((1u << e_lo) - 1u);
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                const uint32_t lo16 = 0u - ((keep >> (2 * j)) & 1u), hi16 = 0u - ((keep >> (2 * j + 1)) & 1u);
                d4[j] &= (lo16 & 0x0000ffffu) | (hi16 << 16);
              }
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j) d4[j] = (j >= e_lo && j < e_hi) ? d4[j] : 0u;
            }
            w.x = d4[0]; w.y = d4[1]; w.z = d4[2]; w.w = d4[3];
          }
          v = w;
        } else {
          alignas(16) T tmp[E];
#pragma unroll
          for (int e = 0; e < E; ++e) tmp[e] = (e >= e_lo && e < e_hi) ? src[x0 + e * p.sw] : T(0);
          v = *reinterpret_cast<u32x4*>(tmp);
        }
      }
    }
    reg[u] = v;
  }
}

template <typename T>
__device__ __forceinline__ void store_panel(AK_LDS unsigned char* plane, const u32x4 (&reg)[CH], const ChunkTab& tab,
                                            int nch) {
#pragma unroll
  for (int u = 0; u < CH; ++u)
    if (u < nch)
      *reinterpret_cast<AK_LDS u32x4*>(plane + static_cast<uint32_t>(tab.pk[u] >> 12) * 16u) = reg[u];
}

template <typename T, int TI>
struct Frags;
template <int TI>
struct Frags<uint16_t, TI> { bf16x8 a[TI], b[TI]; };
template <int TI>
struct Frags<float, TI> { floatx4 a[TI][2], b[TI][2]; };

template <typename T, int TI>
__device__ __forceinline__ void read_frags(Frags<T, TI>& f, AK_LDS const unsigned char* pI, AK_LDS const unsigned char* pJ,
                                           const uint32_t (&bI)[TI], const uint32_t (&bJ)[TI], uint32_t off) {
#pragma unroll
  for (int a = 0; a < TI; ++a) {
    if constexpr (sizeof(T) == 2) {
      f.a[a] = *reinterpret_cast<AK_LDS const bf16x8*>(pI + bI[a] + off);
    } else {
      f.a[a][0] = *reinterpret_cast<AK_LDS const floatx4*>(pI + bI[a] + off);
      f.a[a][1] = *reinterpret_cast<AK_LDS const floatx4*>(pI + bI[a] + off + 16);
    }
  }
#pragma unroll
  for (int b = 0; b < TI; ++b) {
    if constexpr (sizeof(T) == 2) {
      f.b[b] = *reinterpret_cast<AK_LDS const bf16x8*>(pJ + bJ[b] + off);
    } else {
      f.b[b][0] = *reinterpret_cast<AK_LDS const floatx4*>(pJ + bJ[b] + off);
      f.b[b][1] = *reinterpret_cast<AK_LDS const floatx4*>(pJ + bJ[b] + off + 16);
    }
  }
}

template <typename T, int TI>
__device__ __forceinline__ void mma_frags(floatx16 (&acc)[TI][TI], const Frags<T, TI>& f) {
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
      for (int b = 0; b < TI; ++b) acc[a][b] = mfma_bf16(f.a[a], f.b[b], acc[a][b]);
  } else {
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
      for (int a = 0; a < TI; ++a)
#pragma unroll
        for (int b = 0; b < TI; ++b) acc[a][b] = mfma_f32(f.a[a][m >> 2][m & 3], f.b[b][m >> 2][m & 3], acc[a][b]);
  }
}

template <typename T, int TI>
__global__ __launch_bounds__(256, 2) void conv_syrk_kernel(ConvSyrkParams p) {
  constexpr int BT = 64 * TI;
  constexpr int E = Elem<T>::E;
  constexpr uint32_t ES = sizeof(T);
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  AK_LDS unsigned char* lds = (AK_LDS unsigned char*)smem;
  const uint32_t panel_bytes = static_cast<uint32_t>(p.panel_elems) * ES;
  AK_LDS unsigned char* planeI = lds;
  AK_LDS unsigned char* planeJ = lds + panel_bytes;
  AK_LDS unsigned char* zero_unit = lds + 2 * panel_bytes;       // 32 bytes of zeros behind the panels

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = wave >> 1, wc = wave & 1;
  const int g = lane >> 5, l32 = lane & 31;
  int ti, tj;
  decode_upper_tile(blockIdx.x, p.T, ti, tj);
  const bool diag = (ti == tj);
  const int64_t i0 = static_cast<int64_t>(ti) * BT, j0 = static_cast<int64_t>(tj) * BT;
  const T* __restrict__ x = static_cast<const T*>(p.x);

  auto chan_range = [&](int64_t r0, int& c_lo, int& nc) {
    int64_t last = r0 + BT - 1;
    if (last > p.d - 1) last = p.d - 1;
    c_lo = static_cast<int>(fastdiv(static_cast<uint32_t>(r0), p.mKK, p.KK));
    nc = static_cast<int>(fastdiv(static_cast<uint32_t>(last), p.mKK, p.KK)) - c_lo + 1;
  };
  int cI, ncI, cJ, ncJ;
  chan_range(i0, cI, ncI);
  chan_range(j0, cJ, ncJ);
  if (diag) planeJ = planeI;

  auto frag_base = [&](int64_t row, int c_lo) {     // byte offset of row i's first input row inside its panel
    if (row > p.d - 1) row = p.d - 1;
    const uint32_t i = static_cast<uint32_t>(row);
    const uint32_t c = fastdiv(i, p.mKK, p.KK);
    const uint32_t rem = i - c * p.KK;
    const uint32_t ky = fastdiv(rem, p.mKw, p.kw);
    const uint32_t kx = rem - ky * p.kw;
    return ((c - c_lo) * p.CS + kx * p.PS + ky * p.RS) * ES;
  };
  uint32_t baseI[TI], baseJ[TI];
#pragma unroll
  for (int a = 0; a < TI; ++a) baseI[a] = frag_base(i0 + 32 * TI * wr + 32 * a + l32, cI);
#pragma unroll
  for (int b = 0; b < TI; ++b) baseJ[b] = frag_base(j0 + 32 * TI * wc + 32 * b + l32, cJ);

  if (tid < 8) *reinterpret_cast<AK_LDS uint32_t*>(zero_unit + 4 * tid) = 0u;

  // staging tables
  const int CPR = p.WC / E;
  const int row0 = static_cast<int>(fastdiv(tid, p.mCPR, CPR));
  const int q0 = (tid - row0 * CPR) * E;
  const int kwRI = p.kw * p.RI;
  const int nchI = row0 < p.RP ? (ncI * kwRI - row0 + p.RP - 1) / p.RP : 0;   // chunks this thread stages
  const int nchJ = (diag || row0 >= p.RP) ? 0 : (ncJ * kwRI - row0 + p.RP - 1) / p.RP;
  ChunkTab tabI, tabJ;
  build_tab(tabI, p, cI, ncI, row0, q0, E);
  build_tab(tabJ, p, cJ, ncJ, row0, q0, E);

  floatx16 acc[TI][TI];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TI; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  const int64_t s_begin = static_cast<int64_t>(blockIdx.y) * p.stages_per_split;
  int64_t s_end = s_begin + p.stages_per_split;
  if (s_end > p.total_stages) s_end = p.total_stages;
  const int RBCB = p.RB * p.CB;
  const int64_t img_elems = p.C * p.H * p.W;

  auto geom = [&](int64_t s, StageGeom& sg, int& R_eff) {
    const uint32_t s32 = static_cast<uint32_t>(s);
    const uint32_t n = fastdiv(s32, p.mRBCB, RBCB);
    const uint32_t t2 = s32 - n * RBCB;
    const uint32_t rb = fastdiv(t2, p.mCB, p.CB);
    const uint32_t cb = t2 - rb * p.CB;
    const int oy0 = rb * p.R, ox0 = cb * p.WC;
    R_eff = min(p.R, p.Ho - oy0);
    sg.iy0 = oy0 * p.sh - p.ph;
    sg.img = static_cast<int64_t>(n) * img_elems + static_cast<int64_t>(sg.iy0) * p.W;
    sg.xq = ox0 * p.sw - p.pw;
    sg.W_eff = min(p.WC, p.Wo - ox0);
    sg.RI_eff = (R_eff - 1) * p.sh + p.kh;
  };

  // per-lane walk over the k-units of a stage: lanes with g = 0 take units 0, 2, 4, ..., g = 1 take 1, 3, ...
  const uint32_t unit_bytes = 8 * ES;
  const uint32_t row_bytes = static_cast<uint32_t>(p.sh * p.RS) * ES;
  const uint32_t row_jump = row_bytes - static_cast<uint32_t>(p.U) * unit_bytes;
  uint32_t u_first, off_first;       // unit g of a stage
  if (g < p.U) { u_first = g; off_first = g * unit_bytes; }
  else { u_first = 0; off_first = row_bytes; }   // U == 1: unit 1 is row 1, column 0

  u32x4 regI[CH], regJ[CH];
  StageGeom sg;
  int R_cur = 0, R_next = 0;
  if (s_begin < s_end) {
    geom(s_begin, sg, R_next);
    fetch_panel<T>(regI, tabI, p, x, sg, q0, nchI);
    if (!diag) fetch_panel<T>(regJ, tabJ, p, x, sg, q0, nchJ);
  }
  for (int64_t s = s_begin; s < s_end; ++s) {
    R_cur = R_next;
    __syncthreads();                       // every wave is done reading the previous stage
    store_panel<T>(planeI, regI, tabI, nchI);
    if (!diag) store_panel<T>(planeJ, regJ, tabJ, nchJ);
    __syncthreads();
    if (s + 1 < s_end) {                   // next stage's global loads fly while this stage computes
      geom(s + 1, sg, R_next);
      fetch_panel<T>(regI, tabI, p, x, sg, q0, nchI);
      if (!diag) fetch_panel<T>(regJ, tabJ, p, x, sg, q0, nchJ);
    }

    const int nunits = R_cur * p.U;
    const int nfull = nunits >> 1;         // k-steps in which both lane halves have a real unit
    uint32_t u = u_first, off = off_first;
    auto advance = [&]() {                 // two units further along this lane's walk
      u += 2;
      off += 2 * unit_bytes;
      if (u >= static_cast<uint32_t>(p.U)) {
        u -= p.U;
        off += row_jump;
        if (u >= static_cast<uint32_t>(p.U)) { u -= p.U; off += row_jump; }   // U == 1
      }
    };
    Frags<T, TI> f0, f1;                   // ping-pong: the reads of one fly during the MFMAs of the other
    if (nfull > 0) read_frags<T, TI>(f0, planeI, planeJ, baseI, baseJ, off);
    int t = 0;
    for (; t + 2 <= nfull; t += 2) {
      advance();
      read_frags<T, TI>(f1, planeI, planeJ, baseI, baseJ, off);
      mma_frags<T, TI>(acc, f0);
      advance();
      if (t + 2 < nfull) read_frags<T, TI>(f0, planeI, planeJ, baseI, baseJ, off);
      mma_frags<T, TI>(acc, f1);
    }
    if (t < nfull) {                       // odd count: f0 holds the last full step
      advance();
      mma_frags<T, TI>(acc, f0);
    }
    if (nunits & 1) {                      // last unit: the g = 1 half multiplies zeros
      Frags<T, TI> tail;
      AK_LDS const unsigned char* tI = g ? zero_unit : planeI + off;
      AK_LDS const unsigned char* tJ = g ? zero_unit : planeJ + off;
      uint32_t zI[TI], zJ[TI];
#pragma unroll
      for (int a = 0; a < TI; ++a) zI[a] = g ? 0u : baseI[a];
#pragma unroll
      for (int b = 0; b < TI; ++b) zJ[b] = g ? 0u : baseJ[b];
      read_frags<T, TI>(tail, tI, tJ, zI, zJ, 0u);
      mma_frags<T, TI>(acc, tail);
    }
  }

  if (p.nsplit == 1) {
    syrk_epilogue<TI, TI>(acc, p.A, p.lda, p.d, i0 + 32 * TI * wr, j0 + 32 * TI * wc, diag, p.alpha, p.beta, lane);
  } else {
    store_partial<TI, TI>(acc, p.ws + (static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (BT * BT), tid);
  }
}

// Host-side geometry shared by the launch and the workspace query.
struct ConvPlan {
  ConvSyrkParams p;
  int BT;
  size_t lds_bytes;
  int64_t ntiles;
  size_t ws_need;
};

static int tile_rows_for(int64_t d) { return d <= 64 ? 64 : 128; }

// Number of rows, over all groups of 8 consecutive rows i, that share a 16-byte bank group with an earlier
// row of their group, for LDS strides given in 16-byte units.
static int bank_conflicts(int KK, int kw, int rsu, int psu, int csu) {
  int bad = 0;
  for (int t = 0; t < KK; ++t) {
    int seen = 0;
    for (int e = 0; e < 8; ++e) {
      const int i = 8 * t + e, c = i / KK, rem = i % KK, ky = rem / kw, kx = rem % kw;
      const int unit = (c * csu + kx * psu + ky * rsu) & 7;
      if (seen & (1 << unit)) ++bad;
      seen |= 1 << unit;
    }
  }
  return bad;
}

// Picks paddings (in 16-byte units) for the row / plane / channel strides: fewest conflicts, then smallest.
static void pick_strides(int KK, int kw, int RI, int wcu, int& rsu, int& psu, int& csu) {
  int best = 1 << 30;
  for (int p0 = 0; p0 < 8; ++p0)
    for (int p1 = 0; p1 < 8; ++p1)
      for (int p2 = 0; p2 < 8; ++p2) {
        const int r = wcu + p0, ps = RI * r + p1, cs = kw * ps + p2;
        const int score = bank_conflicts(KK, kw, r, ps, cs) * 100000 + cs;
        if (score < best) { best = score; rsu = r; psu = ps; csu = cs; }
      }
}

static bool build_plan(ConvPlan& plan, int esize, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                       int sw, int ph, int pw) {
  ConvSyrkParams& p = plan.p;
  const int BT = tile_rows_for(C * kh * kw);
  plan.BT = BT;
  bool flat = false;
  if (kh == 1 && kw == 1 && ph == 0 && pw == 0 && sh == 1 && sw == 1) {  // positions are contiguous: flatten
    W = H * W;
    H = 1;
    flat = true;
  }
  const int64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
  if (Ho <= 0 || Wo <= 0) return false;
  if (kw > 15 || kh > 255) return false;                 // table packing
  p.N = N; p.C = C; p.H = H; p.W = W;
  p.total_elems = N * C * H * W;
  if (C * H * W >= (1ll << 31)) return false;
  p.kh = kh; p.kw = kw; p.sh = sh; p.sw = sw; p.ph = ph; p.pw = pw;
  p.Ho = static_cast<int>(Ho); p.Wo = static_cast<int>(Wo);
  p.KK = kh * kw;
  p.d = C * p.KK;
  int ncmax = (BT - 1 + p.KK - 1) / p.KK + 1;
  if (ncmax > C) ncmax = static_cast<int>(C);
  p.NCmax = ncmax;
  const int E = 16 / esize;
  const size_t budget = 80 * 1024 - 64;     // two work groups per CU
  const int wo8 = static_cast<int>(((Wo + 7) / 8) * 8);
  int WC = 0, R = 0, rsu = 0, psu = 0, csu = 0;
  const int cands[5] = {128, 64, 32, 16, 8};
  for (int ci = (flat && esize == 2) ? 0 : 1; ci < 5 && R == 0; ++ci) {
    int wc = cands[ci] < wo8 ? cands[ci] : wo8;
    {  // equal column chunks: the padding of the last chunk is spread out
      const int64_t ncb = (Wo + wc - 1) / wc;
      wc = static_cast<int>((((Wo + ncb - 1) / ncb) + 7) / 8 * 8);
    }
    const int wcu = wc / E;
    const int rp = 256 / wcu;
    for (int cand = 1; cand <= Ho && cand * wc <= 1024 && (cand - 1) * sh + kh <= 254; ++cand) {
      const int RI = (cand - 1) * sh + kh;
      const int64_t rows = static_cast<int64_t>(ncmax) * kw * RI;
      int a, b, c;
      pick_strides(p.KK, kw, RI, wcu, a, b, c);
      const size_t bytes = 2ull * ncmax * c * 16;
      // chunk slots per thread, LDS budget, and the 20-bit LDS offset field of the chunk table
      if (rows <= static_cast<int64_t>(CH) * rp && bytes <= budget && static_cast<int64_t>(ncmax) * c < (1 << 19))
        R = cand;
      else
        break;
    }
    if (R > 0) WC = wc;
  }
  if (R == 0) return false;
  {  // equal-sized row blocks: no short last block
    const int64_t nrb = (Ho + R - 1) / R;
    R = static_cast<int>((Ho + nrb - 1) / nrb);
  }
  p.WC = WC;
  p.U = WC / 8;
  p.R = R;
  p.RI = (R - 1) * sh + kh;
  pick_strides(p.KK, kw, p.RI, WC / E, rsu, psu, csu);
  p.RS = rsu * E; p.PS = psu * E; p.CS = csu * E;
  p.panel_elems = ncmax * p.CS;
  plan.lds_bytes = 2ull * p.panel_elems * esize + 64;
  if (plan.lds_bytes > 160 * 1024) return false;
  p.RB = static_cast<int>((Ho + R - 1) / R);
  p.CB = static_cast<int>((Wo + WC - 1) / WC);
  p.total_stages = N * p.RB * p.CB;
  if (p.total_stages >= (1ll << 31) || p.d >= (1ll << 24)) return false;
  if (p.total_stages * p.RB * p.CB >= (1ll << 32)) return false;   // exactness of the magic division
  const int64_t Tn = (p.d + BT - 1) / BT;
  p.T = static_cast<int>(Tn);
  plan.ntiles = Tn * (Tn + 1) / 2;
  const int64_t ksteps_per_stage = (static_cast<int64_t>(R) * WC + 31) / 32;
  int nsplit = pick_nsplit(plan.ntiles, p.total_stages * ksteps_per_stage);
  if (nsplit > p.total_stages) nsplit = static_cast<int>(p.total_stages);
  if (nsplit < 1) nsplit = 1;
  p.stages_per_split = (p.total_stages + nsplit - 1) / nsplit;
  if (p.stages_per_split < 1) p.stages_per_split = 1;
  nsplit = static_cast<int>((p.total_stages + p.stages_per_split - 1) / p.stages_per_split);
  if (nsplit < 1) nsplit = 1;
  p.nsplit = nsplit;
  plan.ws_need = nsplit > 1 ? static_cast<size_t>(nsplit) * plan.ntiles * BT * BT * sizeof(float) : 0;
  const int CPR = WC / E;
  p.RP = 256 / CPR;
  {
    const int kwRI = kw * p.RI;
    p.dcl = p.RP / kwRI;
    const int rem = p.RP - p.dcl * kwRI;
    p.dkx = rem / p.RI;
    p.dr = rem - p.dkx * p.RI;
  }
  p.mKK = make_magic(p.KK); p.mKw = make_magic(kw); p.mRI = make_magic(p.RI);
  p.mKwRI = make_magic(kw * p.RI); p.mCPR = make_magic(CPR); p.mCB = make_magic(p.CB);
  p.mRBCB = make_magic(p.RB * p.CB);
  return true;
}

// Plans depend on the geometry only and cost a stride search: keep them (read-mostly, mutex protected).
struct PlanKey {
  int64_t v[12];
  bool operator<(const PlanKey& o) const {
    for (int i = 0; i < 12; ++i)
      if (v[i] != o.v[i]) return v[i] < o.v[i];
    return false;
  }
};

static bool make_plan(ConvPlan& plan, int esize, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                      int sw, int ph, int pw) {
  static std::mutex mu;
  static std::map<PlanKey, std::pair<bool, ConvPlan>> cache;
  const PlanKey key{{esize, N, C, H, W, kh, kw, sh, sw, ph, pw, 0}};
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = cache.find(key);
    if (it != cache.end()) {
      plan = it->second.second;
      return it->second.first;
    }
  }
  ConvPlan fresh{};
  const bool ok = build_plan(fresh, esize, N, C, H, W, kh, kw, sh, sw, ph, pw);
  {
    std::lock_guard<std::mutex> lock(mu);
    if (cache.size() > 4096) cache.clear();
    cache[key] = std::make_pair(ok, fresh);
  }
  plan = fresh;
  return ok;
}

template <typename T, int TI>
static int launch_conv_syrk_t(ConvPlan& plan, hipStream_t stream) {
  auto kern = conv_syrk_kernel<T, TI>;
  if (plan.lds_bytes > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(plan.lds_bytes)) != hipSuccess)
      return AK_ERR_LAUNCH;
  }
  dim3 grid(static_cast<unsigned>(plan.ntiles), static_cast<unsigned>(plan.p.nsplit));
  hipLaunchKernelGGL(kern, grid, dim3(256), plan.lds_bytes, stream, plan.p);
  if (plan.p.nsplit > 1)
    hipLaunchKernelGGL((syrk_finalize_kernel<TI, TI>), dim3(static_cast<unsigned>(plan.ntiles), 4 * TI * TI), dim3(256), 0,
                       stream, static_cast<const float*>(plan.p.ws), plan.p.nsplit, plan.p.T, plan.p.A, plan.p.lda,
                       plan.p.d, plan.p.alpha, plan.p.beta);
  return check_launch();
}

template <typename T>
static int launch_conv_syrk(ConvPlan& plan, hipStream_t stream) {
  return plan.BT == 64 ? launch_conv_syrk_t<T, 1>(plan, stream) : launch_conv_syrk_t<T, 2>(plan, stream);
}

}  // namespace ak

extern "C" size_t ak_conv_syrk_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw,
                                        int ph, int pw) {
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 || ph < 0 || pw < 0) return 0;
  const size_t patch = ak::conv_patch_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw);
  if (patch > 0) return patch;
  ak::ConvPlan a, b;
  size_t need = ak::conv_corr_f32_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw);
  if (ak::make_plan(a, 2, N, C, H, W, kh, kw, sh, sw, ph, pw) && a.ws_need > need) need = a.ws_need;
  if (ak::make_plan(b, 4, N, C, H, W, kh, kw, sh, sw, ph, pw) && b.ws_need > need) need = b.ws_need;
  return need;
}

extern "C" int ak_conv_syrk(const void* x, int dtype, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh,
                            int sw, int ph, int pw, float alpha, float beta, float* A, int64_t lda, void* ws,
                            size_t ws_bytes, ak_stream_t stream) {
  if (x == nullptr || A == nullptr || N <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || sh <= 0 ||
      sw <= 0 || ph < 0 || pw < 0)
    return AK_ERR_ARG;
  if (dtype != AK_BF16 && dtype != AK_F32 && dtype != AK_F32_AS_BF16) return AK_ERR_ARG;
  if (!ak::syrk_beta_ok(beta, C * kh * kw, lda)) return AK_ERR_UNSUPPORTED;
  {  // few input channels: the window kernel
    const int rc = ak::conv_patch_syrk(x, dtype, C * H * W, H * W, W, 1, N, C, H, W, kh, kw, sh, sw, ph, pw, alpha, beta,
                                       A, lda, ws, ws_bytes, static_cast<hipStream_t>(stream));
    if (rc != AK_ERR_UNSUPPORTED) return rc;
  }
  if (dtype == AK_F32_AS_BF16) return AK_ERR_UNSUPPORTED;      // rounding on the fly is the window kernel's
  if (dtype == AK_F32) {
    // 3 x 3, stride 1, padding 1: shifted correlations of three bf16 planes of the input
    const int rc = ak::conv_corr_syrk_f32(static_cast<const float*>(x), N, C, H, W, kh, kw, sh, sw, ph, pw, alpha, beta, A,
                                          lda, ws, ws_bytes, static_cast<hipStream_t>(stream));
    if (rc != AK_ERR_UNSUPPORTED) return rc;
  }
  ak::ConvPlan plan;
  if (!ak::make_plan(plan, dtype == AK_BF16 ? 2 : 4, N, C, H, W, kh, kw, sh, sw, ph, pw)) return AK_ERR_UNSUPPORTED;
  if (lda < plan.p.d) return AK_ERR_ARG;
  if (plan.ws_need > 0 && (ws == nullptr || ws_bytes < plan.ws_need)) return AK_ERR_WORKSPACE;
  plan.p.x = x; plan.p.alpha = alpha; plan.p.beta = beta; plan.p.A = A; plan.p.lda = lda;
  plan.p.ws = static_cast<float*>(ws);
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == AK_BF16 ? ak::launch_conv_syrk<uint16_t>(plan, s) : ak::launch_conv_syrk<float>(plan, s);
}
