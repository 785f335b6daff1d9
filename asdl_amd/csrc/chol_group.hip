// out_m <- (A_m + lam_m I)^-1 for many symmetric positive definite fp32 matrices of DIFFERENT sizes in one call.
//
// Per matrix (work matrix W, lower triangle) a right-looking blocked Cholesky that keeps the inverses of its 128 x 128
// diagonal blocks, then the triangular inverse by levels, then out = M^T M (cg_right_looking below):
//   for every diagonal block k:  leaf: W_kk -> M_kk = L_kk^-1 (one work group, in the LDS: chol_leaf.hpp);
//                                panel: L21 = A21 M_kk^T;  update: A22 -= L21 L21^T
//   for every level of a balanced tree over the blocks:  T2 = L21 M11;  M21 = -M22 T2
// d^3 FLOP in total, like POTRF + POTRI.  Explicit inverses are taken of 128 x 128 diagonal blocks only, so a panel is
// as accurate as a triangular solve with a block of that size (measured against fp64 on rank-deficient factors: 1.4-1.7
// times the error of LAPACK's fp32 potrf + potri; a recursion that multiplied by the inverse of a whole half was at 3-8).
//
// The per-matrix sequences of steps (leaf | products) of ALL matrices are merged into one sequence of "super-steps":
// super-step s holds, for every matrix whose next step has the type chosen for s, that step.  One launch per
// super-step: a grouped leaf launch (one work group per diagonal block) or a grouped product launch (one work group
// per 128 x 128 tile of any product of the step, split-operand MFMA tile of gemm_x3.hpp, descriptor found through a
// tile -> product map).  The longest chain (the largest matrix) sets the number of launches; the work of all smaller
// matrices runs in the shadow of its steps.  ResNet-50 (108 factors, 13 sizes): 121 launches.
//
// The plan (descriptor tables, launch sequence) depends on the sizes only; every address in it is an offset into the
// workspace.  The caller builds it once per size set on the host (ak_chol_group_plan), keeps a device copy, and
// passes both to every call.
//
// Matrices are padded to a multiple of 4 columns with an identity block (the padded rows and columns drop out of the
// result), which keeps every operand of the split kernel 16-byte aligned.  Only the lower triangle of the input is
// read; the strictly upper 128-blocks of W are never touched.
#include <algorithm>
#include <cstring>
#include <vector>
#include "gemm_f32.hpp"
#include "chol_leaf.hpp"

namespace ak {

constexpr int64_t CG_MAGIC = 0x3247524c4f4843ll;     // "CHOLGR2"
constexpr int CG_COPY = 0, CG_LEAF = 1, CG_PROD = 2;
constexpr int CG_FLAG_TRANSA = 1, CG_FLAG_TRANSB = 2, CG_FLAG_OUT_USER = 4;
// What an operand of a product holds, for the fp16-piece products (bits 4-5 of CgProd::flags: A, bits 6-7: B).  With
// a = the largest diagonal element of A + lam I, every element is bounded in magnitude: a block of the (updated)
// matrix by a, of its Cholesky factor L by sqrt(a), of M = L^-1 by 1 / sqrt(lam), of L21 L11^-1 by sqrt(a / lam).
constexpr int CG_KIND_W = 0, CG_KIND_L = 1, CG_KIND_M = 2, CG_KIND_T2 = 3;
constexpr int CG_SCALE_FLOATS = 8;                    // per matrix: the four scales, the fp16 switch, padding
#ifdef AK_TUNING_HOOKS
static float CG_HALF_MAX_COND = 65536.f;              // tuning builds: ak_debug_set_chol_half_max_cond
#else
constexpr float CG_HALF_MAX_COND = 65536.f;           // a / lam beyond 2^16: the matrix keeps the bf16 three-piece products
#endif
constexpr int CG_GROUP = 4;                           // block columns whose updates of the trailing matrix are merged
constexpr int CG_COPY_ROWS = 8;                       // rows of W one work group of the copy-in kernel writes

struct CgHeader {
  int64_t magic;
  int64_t total_bytes;
  int64_t ws_floats;
  int64_t scales_off;       // floats from the workspace base: CG_SCALE_FLOATS per matrix
  int64_t mats_off, steps_off, leaves_off, prods_off, map_off;     // byte offsets of the tables inside the plan
  int32_t count, nsteps, nleaves, nprods;
  int32_t copy_blocks, ntiles;
};

struct CgMat {
  int64_t w_off;            // work matrix [dp, dp], offset in floats from the workspace base
  int32_t d, dp;
  int32_t first_copy_block, pad0;
};

struct CgStep {
  int32_t type, first, count, grid;
  int32_t first_tile, pad0;     // products: where the step's tile -> product map starts
};

struct CgLeafTask {
  int64_t blk_off;          // the diagonal block, offset in floats from the workspace base
  int32_t mat, lo, n, ld, d, pad0;
};

struct CgProd {
  int64_t a_off, b_off, c_off;
  int32_t lda, ldb, ldc;
  int32_t M, N, K;
  int32_t flags, kmode, tile_mode;
  float alpha, beta;
  int32_t mat;
  int32_t first_tile, tiles_m, tiles_n;
};

struct CgArgs {
  const unsigned char* plan;        // device copy of the plan
  float* ws;
  const float* const* A_list;
  float* const* out_list;
  const float* lam;
  const int* skip;
  int* info;
  int lam_stride, skip_stride;
  float* scales;                    // ws + scales_off
};

__device__ __forceinline__ bool cg_skipped(const CgArgs& a, int mat) {
  return a.skip != nullptr && a.skip[static_cast<int64_t>(mat) * a.skip_stride] == 0;
}

// W_m <- lower(A_m) + lam_m I, padded rows carry the identity; info_m <- 0.  One work group per CG_COPY_ROWS rows of
// one matrix (bisection on first_copy_block); a row is read and written up to its diagonal element only.
static __global__ __launch_bounds__(256) void cg_copy_in_kernel(CgArgs a, int count) {
  const CgHeader* __restrict__ h = reinterpret_cast<const CgHeader*>(a.plan);
  const CgMat* __restrict__ mats = reinterpret_cast<const CgMat*>(a.plan + h->mats_off);
  const int w = blockIdx.x;
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (mats[mid].first_copy_block <= w) lo = mid;
    else hi = mid - 1;
  }
  const CgMat m = mats[lo];
  if (cg_skipped(a, lo)) return;
  const int r0 = (w - m.first_copy_block) * CG_COPY_ROWS;
  if (r0 == 0 && threadIdx.x == 0) a.info[lo] = 0;
  const float* __restrict__ A = a.A_list[lo];
  float* __restrict__ W = a.ws + m.w_off;
  const float l = a.lam[static_cast<int64_t>(lo) * a.lam_stride];
  const bool vec = (m.d % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
#pragma unroll 1
  for (int e = 0; e < CG_COPY_ROWS; ++e) {
    const int r = r0 + e;
    if (r >= m.dp) break;
    float* __restrict__ dst = W + static_cast<int64_t>(r) * m.dp;
    if (r >= m.d) {
      // padding: a diagonal block that drops out of the result.  Its value lam (1 when lam <= 0) stays inside the
      // magnitude bounds the fp16-piece products scale their operands by (lam <= a, 1 / sqrt(lam) for the inverse).
      const float pad = l > 0.f ? l : 1.f;
      for (int c = threadIdx.x; c <= r; c += 256) dst[c] = (c == r) ? pad : 0.f;
      continue;
    }
    const float* __restrict__ src = A + static_cast<int64_t>(r) * m.d;
    if (vec) {
      for (int c = 4 * threadIdx.x; c <= r; c += 1024) {
        floatx4 v = *reinterpret_cast<const floatx4*>(src + c);
        if (r >= c && r < c + 4) v[r - c] += l;
        *reinterpret_cast<floatx4*>(dst + c) = v;       // the elements right of the diagonal are never read
      }
    } else {
      for (int c = threadIdx.x; c <= r; c += 256) dst[c] = src[c] + ((c == r) ? l : 0.f);
    }
  }
}

// Per matrix: the powers of two that bring each kind of operand into the range of fp16 (largest possible magnitude
// -> (2^13, 2^14]), from a = max_i (A_ii + lam) and lam; and whether the matrix takes the fp16-piece products at
// all: a > 0, lam > 0 and a / lam <= 2^16 (elements that are much smaller than their kind's bound lose relative, not
// absolute accuracy; within that ratio the elements that matter keep 22 bits, and the condition number, at most d a / lam,
// leaves the two bits the fp16 pieces have less than fp32 to spare before the factorization breaks down).  One work group
// per matrix.
static __global__ __launch_bounds__(256) void cg_scale_kernel(CgArgs a, int count, float max_cond) {
  __shared__ float red[4];
  const int m = blockIdx.x;
  const CgHeader* __restrict__ h = reinterpret_cast<const CgHeader*>(a.plan);
  const CgMat cm = reinterpret_cast<const CgMat*>(a.plan + h->mats_off)[m];
  float* __restrict__ sc = a.scales + static_cast<int64_t>(m) * CG_SCALE_FLOATS;
  float amax = -3.0e38f;
  const bool live = !cg_skipped(a, m);
  if (live) {
    const float* __restrict__ A = a.A_list[m];
    for (int i = threadIdx.x; i < cm.d; i += 256) amax = fmaxf(amax, A[static_cast<int64_t>(i) * cm.d + i]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = amax;
  __syncthreads();
  if (threadIdx.x != 0) return;
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float lam = live ? a.lam[static_cast<int64_t>(m) * a.lam_stride] : 0.f;
  amax += lam;
  const bool half = live && lam > 0.f && amax > 0.f && amax < 3.0e38f && amax <= max_cond * lam;
  float s[4] = {1.f, 1.f, 1.f, 1.f};
  if (half) {
    const float bound[4] = {amax, sqrtf(amax), 1.f / sqrtf(lam), sqrtf(amax / lam)};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      int e;
      frexpf(bound[k], &e);              // bound <= 2^e
      s[k] = ldexpf(1.f, 14 - e);
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) sc[k] = s[k];
  sc[4] = half ? 1.f : 0.f;
}

// One work group (16 waves) per leaf task of the step.  Every table is read with one load that depends on nothing
// but the work group's index: a chain of dependent loads from cold device memory costs a microsecond per link.
static __global__ __launch_bounds__(LEAF_THREADS) void cg_leaf_kernel(CgArgs a, const CgLeafTask* __restrict__ tasks) {
  extern __shared__ __attribute__((aligned(16))) float leaf_smem[];
  const CgLeafTask t = tasks[blockIdx.x];
  const int live = a.skip != nullptr ? a.skip[static_cast<int64_t>(t.mat) * a.skip_stride] : 1;   // used at the end
  const int tid = threadIdx.x;
  leaf_block(a.ws + t.blk_off, t.ld, t.n, leaf_smem, tid);
  const int bad = leaf_bad_pivot(leaf_smem);
  // a bad pivot inside the identity padding cannot happen; one inside the matrix is reported like LAPACK's potrf.
  // A skipped matrix's work area holds whatever the last call left there; its steps still run (they touch nothing
  // but that work area) and report nothing.
  if (tid == 0 && live != 0 && bad != 0 && t.lo + bad <= t.d && a.info[t.mat] == 0) a.info[t.mat] = t.lo + bad;
}

// Tile (ti, tj) number `local` of a product, longest contraction first where the range depends on the tile.
__device__ __forceinline__ void cg_decode_tile(const CgProd& d, int local, int& ti, int& tj) {
  if (d.tile_mode != TILE_ALL) {     // tiles on and below the diagonal, row by row (K_GE_MAXIJ: longest first)
    ti = static_cast<int>((__builtin_sqrtf(8.f * static_cast<float>(local) + 1.f) - 1.f) * 0.5f);
    while ((ti + 1) * (ti + 2) / 2 <= local) ++ti;
    while (ti * (ti + 1) / 2 > local) --ti;
    tj = local - ti * (ti + 1) / 2;
    return;
  }
  switch (d.kmode) {
    case K_LE_J:                     // k <= column tile: last column first
      tj = d.tiles_n - 1 - local / d.tiles_m;
      ti = local % d.tiles_m;
      break;
    case K_GE_J:                     // k >= column tile: first column first
      tj = local / d.tiles_m;
      ti = local % d.tiles_m;
      break;
    case K_LE_I:                     // k <= row tile: last row first
      ti = d.tiles_m - 1 - local / d.tiles_n;
      tj = local % d.tiles_n;
      break;
    default:
      ti = local / d.tiles_n;
      tj = local % d.tiles_n;
      break;
  }
}

// One work group per 128 x 128 tile of any product of the step; tile_map[w] = the product of work group w.
static __global__ __launch_bounds__(256) void cg_prod_kernel(CgArgs a, const CgProd* __restrict__ prods,
                                                             const int32_t* __restrict__ tile_map) {
  __shared__ __attribute__((aligned(16))) unsigned char x3_smem[2 * 3 * X3_PLANE];
  const int w = blockIdx.x;
  const CgProd d = prods[tile_map[w]];
  // only the product that writes the caller's matrix has to respect the skip flag (see cg_leaf_kernel)
  if ((d.flags & CG_FLAG_OUT_USER) && cg_skipped(a, d.mat)) return;
  int ti, tj;
  cg_decode_tile(d, w - d.first_tile, ti, tj);
  GemmParams p;
  p.A = a.ws + d.a_off;
  p.B = a.ws + d.b_off;
  p.C = (d.flags & CG_FLAG_OUT_USER) ? a.out_list[d.mat] : a.ws + d.c_off;
  p.C_list = nullptr;
  p.lda = d.lda; p.ldb = d.ldb; p.ldc = d.ldc;
  p.sA = p.sB = p.sC = 0;
  p.M = d.M; p.N = d.N; p.K = d.K;
  p.transA = (d.flags & CG_FLAG_TRANSA) ? 1 : 0;
  p.transB = (d.flags & CG_FLAG_TRANSB) ? 1 : 0;
  p.alpha = d.alpha; p.beta = d.beta;
  p.kmode = d.kmode; p.tile_mode = d.tile_mode;
  p.active = nullptr; p.active_stride = 0;
  p.split = 3;
  p.chunked = 0;
  p.scaleA = p.scaleB = 1.f;
  const float* __restrict__ sc = a.scales + static_cast<int64_t>(d.mat) * CG_SCALE_FLOATS;
  if (sc[4] != 0.f) {
    // fp16 pieces: two per operand element, three matrix instructions per product instead of six
    p.scaleA = sc[(d.flags >> 4) & 3];
    p.scaleB = sc[(d.flags >> 6) & 3];
    p.alpha = d.alpha / (p.scaleA * p.scaleB);      // powers of two: exact
    gemm_x3_tile<2, false, -1, -1, true>(p, ti, tj, 0, (AK_LDS3 unsigned char*)x3_smem);
  } else {
    gemm_x3_tile<3, false>(p, ti, tj, 0, (AK_LDS3 unsigned char*)x3_smem);
  }
}

// ---- host: the plan ------------------------------------------------------------------------------------------

struct CgOp {                 // one step of one matrix's own sequence
  int type;
  CgLeafTask leaf;
  std::vector<CgProd> prods;
};

static int64_t cg_half(int64_t n) {
  const int64_t nb = (n + LEAF - 1) / LEAF;
  return LEAF * ((nb + 1) / 2);
}

// Floats of the T1 (and of the T2) pool of an n x n range: a node's panels live while its right half is factored.
static int64_t cg_pool(int64_t n) {
  if (n <= LEAF) return 0;
  const int64_t s1 = cg_half(n), s2 = n - s1;
  return std::max(cg_pool(s1), s1 * s2 + cg_pool(s2));
}

static inline int64_t cg_align64(int64_t x) { return (x + 63) / 64 * 64; }

static int64_t cg_tiles(const CgProd& p) {
  const int64_t tm = (p.M + 127) / 128, tn = (p.N + 127) / 128;
  return p.tile_mode == TILE_ALL ? tm * tn : tm * (tm + 1) / 2;
}

static CgProd cg_prod(int mat, int flags, int kind_a, int kind_b, int M, int N, int K, float alpha, int64_t a, int lda,
                      int64_t b, int ldb, float beta, int64_t c, int ldc, int kmode, int tile_mode) {
  CgProd p;
  std::memset(&p, 0, sizeof(p));
  flags |= (kind_a << 4) | (kind_b << 6);
  p.a_off = a; p.b_off = b; p.c_off = c;
  p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.M = M; p.N = N; p.K = K;
  p.flags = flags; p.kmode = kmode; p.tile_mode = tile_mode;
  p.alpha = alpha; p.beta = beta;
  p.mat = mat;
  p.tiles_m = (M + 127) / 128;
  p.tiles_n = (N + 127) / 128;
  return p;
}

// The right-looking sequence of one matrix: for every diagonal block k of 128 columns
//   leaf: W_kk -> M_kk = L_kk^-1;   panel: W[below, k] <- W[below, k] M_kk^T = L[below, k] (in place: every work group
//   reads the 128 x 128 tile it writes, whole, before its epilogue);   update: W22 -= L21 L21^T (lower tiles, K = 128)
// then the triangular inverse by levels of a balanced tree over the blocks (all nodes of one height are independent
// and share two launches):   T2 = L21 M11;  W21 <- M21 = -M22 T2.
// Every product of the factorization phase has as many tiles as the trailing matrix (hundreds for the wide factors).
struct CgNode { int lo, mid, hi, height; };

static int cg_nodes(std::vector<CgNode>& nodes, int lo, int hi) {
  const int n = hi - lo;
  if (n <= LEAF) return 0;
  const int mid = lo + static_cast<int>(cg_half(n));
  const int h = 1 + std::max(cg_nodes(nodes, lo, mid), cg_nodes(nodes, mid, hi));
  nodes.push_back(CgNode{lo, mid, hi, h});
  return h;
}

static void cg_right_looking(std::vector<CgOp>& ops, int mat, int64_t w, int d, int dp, int64_t t2) {
  // Block columns are taken in groups of CG_GROUP: inside a group a block's rank-128 update goes to the remaining
  // columns of the group only; the trailing matrix behind the group gets ONE update with the whole group as its
  // contraction (K up to 128 CG_GROUP), i.e. it is read and written once per group instead of once per block.
  for (int gs = 0; gs < dp; gs += CG_GROUP * LEAF) {
    const int ge = std::min(gs + CG_GROUP * LEAF, dp);
    for (int lo = gs; lo < ge; lo += LEAF) {
      const int n = std::min(LEAF, dp - lo), below = dp - lo - n;
      CgOp leaf;
      leaf.type = CG_LEAF;
      leaf.leaf = CgLeafTask{w + static_cast<int64_t>(lo) * dp + lo, mat, lo, n, dp, d, 0};
      ops.push_back(leaf);
      if (below == 0) break;
      auto at = [&](int r, int c) { return w + static_cast<int64_t>(r) * dp + c; };
      CgOp panel, update;
      panel.type = update.type = CG_PROD;
      panel.prods.push_back(cg_prod(mat, CG_FLAG_TRANSB, CG_KIND_W, CG_KIND_M, below, n, n, 1.f, at(lo + n, lo), dp,
                                    at(lo, lo), dp, 0.f, at(lo + n, lo), dp, K_LE_J, TILE_ALL));
      ops.push_back(panel);
      const int next = lo + n;
      if (next < ge) {
        // the group's remaining columns: the square on the diagonal (lower tiles) and the rows below the group
        const int sq = ge - next, under = dp - ge;
        update.prods.push_back(cg_prod(mat, CG_FLAG_TRANSB, CG_KIND_L, CG_KIND_L, sq, sq, n, -1.f, at(next, lo), dp,
                                       at(next, lo), dp, 1.f, at(next, next), dp, K_FULL, TILE_LOWER));
        if (under > 0)
          update.prods.push_back(cg_prod(mat, CG_FLAG_TRANSB, CG_KIND_L, CG_KIND_L, under, sq, n, -1.f, at(ge, lo), dp,
                                         at(next, lo), dp, 1.f, at(ge, next), dp, K_FULL, TILE_ALL));
      } else {
        // end of the group: the trailing matrix, with the group's ge - gs columns as the contraction
        const int under = dp - ge;
        update.prods.push_back(cg_prod(mat, CG_FLAG_TRANSB, CG_KIND_L, CG_KIND_L, under, under, ge - gs, -1.f, at(ge, gs), dp,
                                       at(ge, gs), dp, 1.f, at(ge, ge), dp, K_FULL, TILE_LOWER));
      }
      ops.push_back(update);
    }
  }
  std::vector<CgNode> nodes;
  const int top = cg_nodes(nodes, 0, dp);
  for (int h = 1; h <= top; ++h) {
    CgOp first, second;
    first.type = second.type = CG_PROD;
    int64_t pool = t2;
    for (const CgNode& nd : nodes) {
      if (nd.height != h) continue;
      const int s1 = nd.mid - nd.lo, s2 = nd.hi - nd.mid;
      const int64_t W11 = w + static_cast<int64_t>(nd.lo) * dp + nd.lo, W21 = w + static_cast<int64_t>(nd.mid) * dp + nd.lo,
                    W22 = w + static_cast<int64_t>(nd.mid) * dp + nd.mid;
      first.prods.push_back(cg_prod(mat, 0, CG_KIND_L, CG_KIND_M, s2, s1, s1, 1.f, W21, dp, W11, dp, 0.f, pool, s1, K_GE_J,
                                    TILE_ALL));
      second.prods.push_back(cg_prod(mat, 0, CG_KIND_M, CG_KIND_T2, s2, s1, s2, -1.f, W22, dp, pool, s1, 0.f, W21, dp,
                                     K_LE_I, TILE_ALL));
      pool += cg_align64(static_cast<int64_t>(s1) * s2);
    }
    ops.push_back(first);
    ops.push_back(second);
  }
}

struct CgPlan {
  CgHeader h;
  std::vector<CgMat> mats;
  std::vector<CgStep> steps;
  std::vector<CgLeafTask> leaves;
  std::vector<CgProd> prods;
  std::vector<int32_t> tile_map;
};

static inline int64_t cg_align(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

static bool cg_dims_ok(const int64_t* dims, int count) {
  if (dims == nullptr || count <= 0 || count > (1 << 20)) return false;
  for (int i = 0; i < count; ++i)
    if (dims[i] <= 0 || dims[i] > 32768) return false;
  return true;
}

static void cg_build(const int64_t* dims, int count, CgPlan& plan) {
  std::vector<std::vector<CgOp>> seq(count);
  int64_t off = 0;
  int copy_blocks = 0;
  plan.mats.resize(count);
  for (int m = 0; m < count; ++m) {
    const int d = static_cast<int>(dims[m]), dp = (d + 3) / 4 * 4;
    const int64_t pool = cg_align(cg_pool(dp), 64);
    CgMat& cm = plan.mats[m];
    cm.w_off = off; cm.d = d; cm.dp = dp; cm.first_copy_block = copy_blocks; cm.pad0 = 0;
    copy_blocks += (dp + CG_COPY_ROWS - 1) / CG_COPY_ROWS;
    const int64_t t1 = off + cg_align(static_cast<int64_t>(dp) * dp, 64), t2 = t1 + pool;
    off = t2 + pool;
    cg_right_looking(seq[m], m, cm.w_off, d, dp, t1);     // the T2 panels of one level: at most dp^2 / 4 + 64 per node
    CgOp fin;
    fin.type = CG_PROD;     // out = M^T M, both triangles
    fin.prods.push_back(cg_prod(m, CG_FLAG_TRANSA | CG_FLAG_OUT_USER, CG_KIND_M, CG_KIND_M, d, d, dp, 1.f, cm.w_off, dp,
                                cm.w_off, dp, 0.f, 0, d, K_GE_MAXIJ, TILE_LOWER_MIRROR));
    seq[m].push_back(fin);
  }
  plan.steps.push_back(CgStep{CG_COPY, 0, count, copy_blocks, 0, 0});
  // Merge: the matrix with the most steps left decides the type of the next super-step; every matrix whose next
  // step has that type takes part.
  std::vector<size_t> cur(count, 0);
  for (;;) {
    int lead = -1;
    size_t most = 0;
    for (int m = 0; m < count; ++m) {
      const size_t left = seq[m].size() - cur[m];
      if (left > most) { most = left; lead = m; }
    }
    if (lead < 0) break;
    const int type = seq[lead][cur[lead]].type;
    CgStep st{type, 0, 0, 0, 0, 0};
    if (type == CG_LEAF) {
      st.first = static_cast<int>(plan.leaves.size());
      for (int m = 0; m < count; ++m)
        if (cur[m] < seq[m].size() && seq[m][cur[m]].type == CG_LEAF) plan.leaves.push_back(seq[m][cur[m]++].leaf);
      st.count = static_cast<int>(plan.leaves.size()) - st.first;
      st.grid = st.count;
    } else {
      std::vector<CgProd> ps;
      for (int m = 0; m < count; ++m)
        if (cur[m] < seq[m].size() && seq[m][cur[m]].type == CG_PROD) {
          for (const CgProd& p : seq[m][cur[m]].prods) ps.push_back(p);
          ++cur[m];
        }
      // longest contraction first: the long tiles start early, the short ones fill the tail
      std::stable_sort(ps.begin(), ps.end(), [](const CgProd& x, const CgProd& y) { return x.K > y.K; });
      int64_t tiles = 0;
      st.first_tile = static_cast<int>(plan.tile_map.size());
      for (size_t i = 0; i < ps.size(); ++i) {
        ps[i].first_tile = static_cast<int>(tiles);
        const int64_t n = cg_tiles(ps[i]);
        tiles += n;
        plan.tile_map.insert(plan.tile_map.end(), static_cast<size_t>(n), static_cast<int32_t>(i));
      }
      st.first = static_cast<int>(plan.prods.size());
      st.count = static_cast<int>(ps.size());
      st.grid = static_cast<int>(tiles);
      plan.prods.insert(plan.prods.end(), ps.begin(), ps.end());
    }
    plan.steps.push_back(st);
  }
  CgHeader& h = plan.h;
  std::memset(&h, 0, sizeof(h));
  h.magic = CG_MAGIC;
  h.scales_off = off;
  off += cg_align(static_cast<int64_t>(count) * CG_SCALE_FLOATS, 64);
  h.ws_floats = off;
  h.count = count;
  h.nsteps = static_cast<int>(plan.steps.size());
  h.nleaves = static_cast<int>(plan.leaves.size());
  h.nprods = static_cast<int>(plan.prods.size());
  h.copy_blocks = copy_blocks;
  h.ntiles = static_cast<int>(plan.tile_map.size());
  int64_t b = cg_align(sizeof(CgHeader), 64);
  h.mats_off = b; b = cg_align(b + plan.mats.size() * sizeof(CgMat), 64);
  h.steps_off = b; b = cg_align(b + plan.steps.size() * sizeof(CgStep), 64);
  h.leaves_off = b; b = cg_align(b + plan.leaves.size() * sizeof(CgLeafTask), 64);
  h.prods_off = b; b = cg_align(b + plan.prods.size() * sizeof(CgProd), 64);
  h.map_off = b; b = cg_align(b + plan.tile_map.size() * sizeof(int32_t), 64);
  h.total_bytes = b;
}

}  // namespace ak

extern "C" size_t ak_chol_group_plan_bytes(const int64_t* dims, int count) {
  if (!ak::cg_dims_ok(dims, count)) return 0;
  ak::CgPlan plan;
  ak::cg_build(dims, count, plan);
  return static_cast<size_t>(plan.h.total_bytes);
}

extern "C" size_t ak_chol_group_ws_bytes(const int64_t* dims, int count) {
  if (!ak::cg_dims_ok(dims, count)) return 0;
  int64_t off = 0;
  for (int m = 0; m < count; ++m) {
    const int64_t dp = (dims[m] + 3) / 4 * 4;
    off += ak::cg_align(dp * dp, 64) + 2 * ak::cg_align(ak::cg_pool(dp), 64);
  }
  off += ak::cg_align(static_cast<int64_t>(count) * ak::CG_SCALE_FLOATS, 64);
  return static_cast<size_t>(off) * sizeof(float);
}

extern "C" int ak_chol_group_plan(const int64_t* dims, int count, void* plan_host, size_t plan_bytes) {
  using namespace ak;
  if (!cg_dims_ok(dims, count) || plan_host == nullptr) return AK_ERR_ARG;
  CgPlan plan;
  cg_build(dims, count, plan);
  if (plan_bytes < static_cast<size_t>(plan.h.total_bytes)) return AK_ERR_WORKSPACE;
  unsigned char* out = static_cast<unsigned char*>(plan_host);
  std::memset(out, 0, static_cast<size_t>(plan.h.total_bytes));
  std::memcpy(out, &plan.h, sizeof(CgHeader));
  std::memcpy(out + plan.h.mats_off, plan.mats.data(), plan.mats.size() * sizeof(CgMat));
  std::memcpy(out + plan.h.steps_off, plan.steps.data(), plan.steps.size() * sizeof(CgStep));
  if (!plan.leaves.empty()) std::memcpy(out + plan.h.leaves_off, plan.leaves.data(), plan.leaves.size() * sizeof(CgLeafTask));
  if (!plan.prods.empty()) std::memcpy(out + plan.h.prods_off, plan.prods.data(), plan.prods.size() * sizeof(CgProd));
  if (!plan.tile_map.empty())
    std::memcpy(out + plan.h.map_off, plan.tile_map.data(), plan.tile_map.size() * sizeof(int32_t));
  return AK_OK;
}

extern "C" int ak_chol_group_plan_launches(const void* plan_host) {
  if (plan_host == nullptr) return AK_ERR_ARG;
  const ak::CgHeader* h = static_cast<const ak::CgHeader*>(plan_host);
  return h->magic == ak::CG_MAGIC ? h->nsteps : AK_ERR_ARG;
}

extern "C" int ak_chol_inv_grouped(const void* plan_host, const void* plan_dev, const float* const* A_list,
                                   float* const* out_list, const float* lam, int lam_stride, const int* skip_flags,
                                   int skip_stride, int* info, void* ws, size_t ws_bytes, ak_stream_t stream) {
  using namespace ak;
  if (plan_host == nullptr || plan_dev == nullptr || A_list == nullptr || out_list == nullptr || lam == nullptr ||
      info == nullptr)
    return AK_ERR_ARG;
  const unsigned char* ph = static_cast<const unsigned char*>(plan_host);
  const CgHeader* h = reinterpret_cast<const CgHeader*>(ph);
  if (h->magic != CG_MAGIC || h->count <= 0 || h->nsteps <= 0) return AK_ERR_ARG;
  if (ws == nullptr || (reinterpret_cast<uintptr_t>(ws) & 255) != 0 ||
      ws_bytes < static_cast<size_t>(h->ws_floats) * sizeof(float))
    return AK_ERR_WORKSPACE;
  static bool leaf_attr_set = false;     // idempotent; a benign race sets it twice at worst
  if (!leaf_attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(cg_leaf_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(LEAF_LDS_BYTES)) != hipSuccess)
      return AK_ERR_LAUNCH;
    leaf_attr_set = true;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  CgArgs a;
  a.plan = static_cast<const unsigned char*>(plan_dev);
  a.ws = static_cast<float*>(ws);
  a.A_list = A_list; a.out_list = out_list;
  a.lam = lam; a.skip = skip_flags; a.info = info;
  a.lam_stride = lam_stride; a.skip_stride = skip_stride;
  a.scales = a.ws + h->scales_off;
  const CgStep* steps = reinterpret_cast<const CgStep*>(ph + h->steps_off);
  for (int i = 0; i < h->nsteps; ++i) {
    const CgStep& st = steps[i];
    if (st.grid <= 0) continue;
    if (st.type == CG_COPY) {
      hipLaunchKernelGGL(cg_copy_in_kernel, dim3(st.grid), dim3(256), 0, s, a, h->count);
      hipLaunchKernelGGL(cg_scale_kernel, dim3(h->count), dim3(256), 0, s, a, h->count, CG_HALF_MAX_COND);
    } else if (st.type == CG_LEAF)
      hipLaunchKernelGGL(cg_leaf_kernel, dim3(st.grid), dim3(LEAF_THREADS), LEAF_LDS_BYTES, s, a,
                         reinterpret_cast<const CgLeafTask*>(a.plan + h->leaves_off) + st.first);
    else
      hipLaunchKernelGGL(cg_prod_kernel, dim3(st.grid), dim3(256), 0, s, a,
                         reinterpret_cast<const CgProd*>(a.plan + h->prods_off) + st.first,
                         reinterpret_cast<const int32_t*>(a.plan + h->map_off) + st.first_tile);
  }
  return check_launch();
}

#ifdef AK_TUNING_HOOKS
// Tuning builds only: the bound a / lam up to which a matrix takes the fp16-piece products (0: never).
extern "C" void ak_debug_set_chol_half_max_cond(float v) { ak::CG_HALF_MAX_COND = v; }
#endif
