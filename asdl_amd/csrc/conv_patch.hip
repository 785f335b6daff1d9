// Conv2d input factor for layers with few input channels (d = C*kh*kw <= 160, e.g. the 3-channel 7x7 stem of
// a ResNet): A = sum over output positions of p p^T, p the (c,ky,kx)-ordered patch, in fp32.
//
// The unfolded matrix has d short rows per position and would be gathered element by element; instead each work
// group stages the input window of a strip of R output rows of one image in LDS once ([c][row][col] planes, zero
// padding materialised) and the lanes of the fp32 matrix instruction read their patch element straight from that
// window: lane l of v_mfma_f32_32x32x2_f32 supplies patch element (32*block + l%32) of position (2*step + l/32).
// The lower 32 x 32 tiles of the (padded) d x d result are spread over the 8 waves; a work group walks over
// several strips and writes one partial per wave and tile slot, summed by a second kernel that also applies
// alpha / beta and mirrors the result.  Input: fp32 with arbitrary element strides (NCHW and NHWC alike).
//
// bf16 input, and fp32 input that is to be rounded to bf16 (AK_F32_AS_BF16), goes to the bf16 matrix instruction
// instead (conv_patch_bf16_kernel): the window is kept as bf16, a lane gathers the same patch element of 8
// consecutive output positions of a row (v_mfma_f32_32x32x16_bf16 wants lane l to hold k = 8*(l/32) .. +7 of row
// l%32, the same layout for both operands of X^T X, so one fragment per 32-block of patch elements serves as
// row operand and as column operand), and every wave keeps ALL lower tiles (15 for d = 147) in its accumulators:
// 5 fragments of 8 two-byte LDS reads feed 15 matrix instructions, which leaves the kernel bound by the matrix
// cores and not by the LDS.  One work group of 4 waves per CU; the four waves' tiles are summed through the LDS
// before they go to the workspace.
#include "common.hpp"

namespace ak {

constexpr int kPatchWaves = 8;
constexpr int kPatchThreads = kPatchWaves * 64;
constexpr int kPatchMaxD = 160;
constexpr size_t kPatchMaxLds = 40 * 1024;   // two work groups per CU
constexpr int kPatchPerThread = static_cast<int>(kPatchMaxLds / 4 / kPatchThreads);   // window elements per thread

struct PatchParams {
  const void* x;
  int64_t sn, sc, sh, sw;        // element strides of x[n][c][iy][ix]
  int N, C, H, W, kh, kw, strh, strw, ph, pw, Ho, Wo;
  int R;                         // output rows per strip
  int strips_per_image, total_strips;
  int PR, PC, RS, plane;         // window rows / columns, LDS row stride, plane size (floats)
  int chan_inner;                // 1: channels are the fastest-moving input axis (NHWC)
  int d, nb, ntiles, tpw, KS;    // 32-blocks, lower tiles, tiles per wave, position slices per tile
  uint32_t mKK, mKw, mPC, mC, mPRPC;
  // bf16 kernel: its window is Q rows of L elements in the order of the input's memory, [window row][column][channel]
  // for a channels-last input (Q = PR, L = PC*C) and [channel][window row][column] otherwise (Q = C*PR, L = PC);
  // LDS row stride RSb.  Patch element (c, ky, kx) of output position (r, ox) of the strip is LDS element
  // c*tap_c + ky*RSb + kx*tap_x + r*strh*RSb + ox*strw*tap_x.
  int G;                         // groups of 8 output positions per output row
  uint32_t mG;
  int Q, L, RSb, tap_c, tap_x, lead, Lvalid;   // lead: window columns left of the input (padding), Lvalid: W*C or W
  uint32_t mL;
  float* ws;                     // [grid][wave][slot][16][64]; bf16 kernel: [grid][tile][16][64]
  int nwg;
  float alpha, beta;
  float* A;
  int64_t lda;
};

__device__ __forceinline__ void patch_tile_blocks(int t, int& bi, int& bj) {
  bi = 0;
  while ((bi + 1) * (bi + 2) / 2 <= t) ++bi;
  bj = t - bi * (bi + 1) / 2;
}

template <typename T>
__device__ __forceinline__ float patch_load(const T* p);
template <>
__device__ __forceinline__ float patch_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float patch_load<uint16_t>(const uint16_t* p) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(*p) << 16);
}

__device__ __forceinline__ float lds_f32(uint32_t byte_addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) float*>(byte_addr);
}

// TWO: every wave holds two tiles (a wave whose second slot is past the last tile repeats tile 0 there; that
// partial is never read).  Four waves per SIMD, i.e. two work groups per CU.
template <typename T, bool TWO>
static __global__ __launch_bounds__(kPatchThreads, 4) void conv_patch_syrk_kernel(PatchParams p) {
  extern __shared__ __attribute__((aligned(16))) float patch_smem[];
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, kk = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // this wave's tiles and position slice
  const int group = wave / p.KS, ks = wave % p.KS;
  int t0 = group * p.tpw, t1 = p.tpw > 1 ? t0 + 1 : -1;
  if (t0 >= p.ntiles) t0 = -1;
  if (t1 >= p.ntiles) t1 = -1;
  int bi0 = 0, bj0 = 0, bi1 = 0, bj1 = 0;
  if (t0 >= 0) patch_tile_blocks(t0, bi0, bj0);
  if (t1 >= 0) patch_tile_blocks(t1, bi1, bj1);               // else tile (0, 0) again
  // LDS offset of this lane's patch element in each of the (up to four) operand blocks
  auto tap_offset = [&](int blk) -> int {
    const uint32_t i = static_cast<uint32_t>(32 * blk + l32);
    if (i >= static_cast<uint32_t>(p.d)) return 0;      // padding rows / columns are computed from any data and never stored
    const uint32_t c = fastdiv(i, p.mKK, p.kh * p.kw);
    const uint32_t rem = i - c * p.kh * p.kw;
    const uint32_t ky = fastdiv(rem, p.mKw, p.kw);
    const uint32_t kx = rem - ky * p.kw;
    return static_cast<int>(c * p.plane + ky * p.RS + kx) * 4;
  };
  const int adv = 2 * p.KS;
  int adv_x, adv_off, wrap_off;
  {
    const int adv_r = adv / p.Wo;
    adv_x = adv - adv_r * p.Wo;
    adv_off = (adv_r * p.strh * p.RS + adv_x * p.strw) * 4;
    wrap_off = (p.strh * p.RS - p.Wo * p.strw) * 4;
  }
  const uint32_t smem_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(patch_smem));
  const int oa0 = tap_offset(bi0), ob0 = tap_offset(bj0), oa1 = tap_offset(bi1), ob1 = tap_offset(bj1);
  floatx16 acc0 = {}, acc1 = {};
  const T* __restrict__ x = static_cast<const T*>(p.x);
  const int window = p.C * p.PR * p.PC;

  // Window elements of one strip, kPatchPerThread per thread, fetched into registers one strip ahead so that the
  // loads are in flight while the previous strip is multiplied.
  float stage[kPatchPerThread];
  auto fetch = [&](int strip) {
    const int n = strip / p.strips_per_image;
    const int iy0 = (strip - n * p.strips_per_image) * p.R * p.strh - p.ph;
    const T* __restrict__ xn = x + static_cast<int64_t>(n) * p.sn;
#pragma unroll 5
    for (int e = 0; e < kPatchPerThread; ++e) {
      const int idx = tid + e * kPatchThreads;
      uint32_t c, pr, pc;
      if (p.chan_inner) {                         // idx = (pr * PC + pc) * C + c
        const uint32_t q = fastdiv(idx, p.mC, p.C);
        c = idx - q * p.C;
        pr = fastdiv(q, p.mPC, p.PC);
        pc = q - pr * p.PC;
      } else {                                    // idx = (c * PR + pr) * PC + pc
        const uint32_t q = fastdiv(idx, p.mPC, p.PC);
        pc = idx - q * p.PC;
        c = fastdiv(q, p.mPRPC, p.PR);
        pr = q - c * p.PR;
      }
      const int iy = iy0 + static_cast<int>(pr), ix = static_cast<int>(pc) - p.pw;
      float v = 0.f;
      if (idx < window && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W)
        v = patch_load<T>(xn + c * p.sc + static_cast<int64_t>(iy) * p.sh + static_cast<int64_t>(ix) * p.sw);
      stage[e] = v;
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int e = 0; e < kPatchPerThread; ++e) {
      const int idx = tid + e * kPatchThreads;
      if (idx >= window) break;
      uint32_t c, pr, pc;
      if (p.chan_inner) {
        const uint32_t q = fastdiv(idx, p.mC, p.C);
        c = idx - q * p.C;
        pr = fastdiv(q, p.mPC, p.PC);
        pc = q - pr * p.PC;
      } else {
        const uint32_t q = fastdiv(idx, p.mPC, p.PC);
        pc = idx - q * p.PC;
        c = fastdiv(q, p.mPRPC, p.PR);
        pr = q - c * p.PR;
      }
      patch_smem[c * p.plane + pr * p.RS + pc] = stage[e];
    }
  };

  if (static_cast<int>(blockIdx.x) < p.total_strips) fetch(blockIdx.x);
  for (int strip = blockIdx.x; strip < p.total_strips; strip += gridDim.x) {
    const int n = strip / p.strips_per_image;
    const int oy0 = (strip - n * p.strips_per_image) * p.R;
    const int rows = min(p.R, p.Ho - oy0);
    __syncthreads();                              // the previous strip's reads are done
    stash();
    __syncthreads();
    if (strip + static_cast<int>(gridDim.x) < p.total_strips) fetch(strip + gridDim.x);
    if (t0 < 0) continue;
    const int npos = rows * p.Wo;
    // This wave multiplies positions 2*(s*KS + ks) + kk, s = 0, 1, ...  Each lane keeps the byte offset of its
    // position inside the window and moves it incrementally; the operands of step s + 1 are read from LDS before
    // the products of step s are issued.
    const int first = 2 * ks;                            // position of the kk = 0 lanes in step 0
    const int nfull = npos - 2 - first >= 0 ? (npos - 2 - first) / adv + 1 : 0;   // steps with both positions
    int ox, off;
    {
      const int pos = first + kk, r = pos / p.Wo;
      ox = pos - r * p.Wo;
      off = (r * p.strh * p.RS + ox * p.strw) * 4;
    }
    auto advance = [&]() {
      ox += adv_x;
      off += adv_off;
      if (ox >= p.Wo) { ox -= p.Wo; off += wrap_off; }
    };
    if (nfull > 0) {
      float a0 = lds_f32(smem_base + oa0 + off), b0 = lds_f32(smem_base + ob0 + off);
      float a1 = lds_f32(smem_base + oa1 + off), b1 = lds_f32(smem_base + ob1 + off);
      for (int st = 1; st < nfull; ++st) {
        advance();
        const float na0 = lds_f32(smem_base + oa0 + off), nb0 = lds_f32(smem_base + ob0 + off);
        const float na1 = lds_f32(smem_base + oa1 + off), nb1 = lds_f32(smem_base + ob1 + off);
        acc0 = mfma_f32(a0, b0, acc0);
        if (TWO) acc1 = mfma_f32(a1, b1, acc1);
        a0 = na0; b0 = nb0; a1 = na1; b1 = nb1;
      }
      acc0 = mfma_f32(a0, b0, acc0);
      if (TWO) acc1 = mfma_f32(a1, b1, acc1);
      advance();
    }
    if (first + nfull * adv < npos) {                    // odd tail: only the kk = 0 lanes hold a position
      const int o = kk == 0 ? off : 0;
      float a0 = lds_f32(smem_base + oa0 + o), b0 = lds_f32(smem_base + ob0 + o);
      float a1 = lds_f32(smem_base + oa1 + o), b1 = lds_f32(smem_base + ob1 + o);
      if (kk != 0) { a0 = 0.f; a1 = 0.f; }
      acc0 = mfma_f32(a0, b0, acc0);
      if (TWO) acc1 = mfma_f32(a1, b1, acc1);
    }
  }
  // partials: [wg][wave][slot][reg][lane]
  float* __restrict__ w = p.ws + ((static_cast<int64_t>(blockIdx.x) * kPatchWaves + wave) * 2) * 1024;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    w[e * 64 + lane] = acc0[e];
    w[1024 + e * 64 + lane] = acc1[e];
  }
}

// One thread per element of a lower 32 x 32 tile: sums the partials of all work groups and position slices.
static __global__ __launch_bounds__(256) void conv_patch_reduce_kernel(PatchParams p) {
  const int t = blockIdx.x >> 2;                       // tile; four blocks of 256 elements each
  const int el = (blockIdx.x & 3) * 256 + threadIdx.x; // reg * 64 + lane
  const int group = t / p.tpw, slot = t - group * p.tpw;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  for (int ksl = 0; ksl < p.KS; ++ksl) {
    const float* __restrict__ w = p.ws + ((static_cast<int64_t>(group * p.KS + ksl)) * 2 + slot) * 1024 + el;
    const int64_t step = static_cast<int64_t>(kPatchWaves) * 2 * 1024;
    int g = 0;
    for (; g + 4 <= p.nwg; g += 4) {
      s[0] += w[(g + 0) * step];
      s[1] += w[(g + 1) * step];
      s[2] += w[(g + 2) * step];
      s[3] += w[(g + 3) * step];
    }
    for (; g < p.nwg; ++g) s[0] += w[g * step];
  }
  const float sum = (s[0] + s[1]) + (s[2] + s[3]);
  int bi, bj;
  patch_tile_blocks(t, bi, bj);
  const int reg = el >> 6, lane = el & 63;
  const int i = 32 * bi + 8 * (reg >> 2) + 4 * (lane >> 5) + (reg & 3);
  const int j = 32 * bj + (lane & 31);
  if (i >= p.d || j >= p.d || (bi == bj && j > i)) return;
  float v = p.alpha * sum;
  float* dst = p.A + static_cast<int64_t>(i) * p.lda + j;
  if (p.beta != 0.f) v += p.beta * *dst;
  *dst = v;
  if (i != j) p.A[static_cast<int64_t>(j) * p.lda + i] = v;
}

// ---- bf16 matrix-instruction variant ------------------------------------------------------------------------
constexpr int kPbWaves = 4;
constexpr int kPbThreads = kPbWaves * 64;
constexpr int kPbStage = 64;                              // window elements per thread
constexpr int kPbMaxWindow = kPbStage * kPbThreads;       // 16384 bf16 elements = 32 KB

__device__ __forceinline__ uint32_t lds_u16(uint32_t byte_addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) uint16_t*>(byte_addr);
}

template <typename T>
__device__ __forceinline__ uint16_t patch_bf16_bits(T v);
template <>
__device__ __forceinline__ uint16_t patch_bf16_bits<uint16_t>(uint16_t v) { return v; }
template <>
__device__ __forceinline__ uint16_t patch_bf16_bits<float>(float v) {      // round to nearest even
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
}

// NB: 32-blocks of patch elements (d <= 32 * NB); the wave holds the NB (NB + 1) / 2 lower tiles.  INNER: channels-last
// input (x[n][iy][ix][c] contiguous).
template <typename T, int NB, bool INNER>
static __global__ __launch_bounds__(kPbThreads) void conv_patch_bf16_kernel(PatchParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char pb_smem[];
  constexpr int NT = NB * (NB + 1) / 2;
  const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, kg = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t smem_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(pb_smem));

  // LDS byte address of this lane's patch element (at output position 0 of the strip) in each 32-block; padding
  // elements (>= d) read element 0: their rows / columns are computed from any data and never stored
  uint32_t tap[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    const uint32_t i = static_cast<uint32_t>(32 * b + l32);
    uint32_t o = 0;
    if (i < static_cast<uint32_t>(p.d)) {
      const uint32_t c = fastdiv(i, p.mKK, p.kh * p.kw);
      const uint32_t rem = i - c * p.kh * p.kw;
      const uint32_t ky = fastdiv(rem, p.mKw, p.kw);
      const uint32_t kx = rem - ky * p.kw;
      o = (c * p.tap_c + ky * p.RSb + kx * p.tap_x) * 2;
    }
    tap[b] = smem_base + o;
  }
  const uint32_t sw2 = static_cast<uint32_t>(p.strw * p.tap_x) * 2;       // bytes between neighbouring output positions
  floatx16 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = floatx16{};
  const T* __restrict__ x = static_cast<const T*>(p.x);
  const int window = p.Q * p.L;
  const int sh = static_cast<int>(p.sh), sw = static_cast<int>(p.sw), sc = static_cast<int>(p.sc);

  // Window elements of one strip, fetched into registers one strip ahead: element idx is column idx % L of window
  // row idx / L.  The index is made opaque to the optimiser, so that row and column are recomputed for every strip
  // instead of being kept in registers for all 64 elements, which the accumulators leave no room for.
  T stage[kPbStage];
  auto fetch = [&](int strip) {
    const int n = strip / p.strips_per_image;
    const int iy0 = (strip - n * p.strips_per_image) * p.R * p.strh - p.ph;
    const T* __restrict__ xn = x + static_cast<int64_t>(n) * p.sn;
#pragma unroll
    for (int e = 0; e < kPbStage; ++e) {
      int idx = tid + e * kPbThreads;
      asm volatile("" : "+v"(idx));
      const uint32_t q = fastdiv(idx, p.mL, p.L);
      const int m = idx - static_cast<int>(q) * p.L - p.lead;      // column of the input row (times C + channel)
      int iy, off;
      if (INNER) {
        iy = iy0 + static_cast<int>(q);
        off = iy * sh + m;
      } else {
        const uint32_t c = fastdiv(q, p.mPRPC, p.PR);
        iy = iy0 + static_cast<int>(q - c * p.PR);
        off = static_cast<int>(c) * sc + iy * sh + m * sw;
      }
      T v = 0;
      if (idx < window && static_cast<uint32_t>(iy) < static_cast<uint32_t>(p.H) &&
          static_cast<uint32_t>(m) < static_cast<uint32_t>(p.Lvalid))
        v = xn[off];
      stage[e] = v;
    }
  };
  auto stash = [&]() {
    uint16_t* const win = reinterpret_cast<uint16_t*>(pb_smem);
#pragma unroll
    for (int e = 0; e < kPbStage; ++e) {
      int idx = tid + e * kPbThreads;
      asm volatile("" : "+v"(idx));
      if (idx >= window) break;
      const uint32_t q = fastdiv(idx, p.mL, p.L);
      win[idx + q * (p.RSb - p.L)] = patch_bf16_bits<T>(stage[e]);
    }
  };
  // the fragments of one step: 8 consecutive output positions (from byte offset off, `valid` of them exist) of this
  // lane's patch element in every 32-block
  auto load_frags = [&](bf16x8 (&f)[NB], uint32_t off, int valid) {
    if (__all(valid == 8)) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint32_t a = tap[b] + off;
        uint32_t w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) w[q] = lds_u16(a + (2 * q) * sw2) | (lds_u16(a + (2 * q + 1) * sw2) << 16);
        f[b] = __builtin_bit_cast(bf16x8, w);
      }
    } else {                                   // end of a row / of the strip: missing positions are zero
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        const uint32_t a = tap[b] + off;
        uint32_t w[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint32_t lo = lds_u16(2 * q < valid ? a + (2 * q) * sw2 : smem_base);
          uint32_t hi = lds_u16(2 * q + 1 < valid ? a + (2 * q + 1) * sw2 : smem_base);
          if (2 * q >= valid) lo = 0;
          if (2 * q + 1 >= valid) hi = 0;
          w[q] = lo | (hi << 16);
        }
        f[b] = __builtin_bit_cast(bf16x8, w);
      }
    }
  };

  if (static_cast<int>(blockIdx.x) < p.total_strips) fetch(blockIdx.x);
  for (int strip = blockIdx.x; strip < p.total_strips; strip += gridDim.x) {
    const int n = strip / p.strips_per_image;
    const int oy0 = (strip - n * p.strips_per_image) * p.R;
    const int rows = min(p.R, p.Ho - oy0);
    __syncthreads();                              // the previous strip's reads are done
    stash();
    __syncthreads();
    if (strip + static_cast<int>(gridDim.x) < p.total_strips) fetch(strip + gridDim.x);
    const int ngroups = rows * p.G;               // groups of 8 positions; a step multiplies two of them
    const int nsteps = (ngroups + 1) >> 1;
    auto locate = [&](int st, uint32_t& off, int& valid) {
      const int g = 2 * st + kg;
      const uint32_t r = fastdiv(g, p.mG, p.G);
      const int ox0 = (g - static_cast<int>(r) * p.G) * 8;
      valid = g < ngroups ? min(8, p.Wo - ox0) : 0;
      off = valid > 0 ? r * p.strh * p.RSb * 2 + ox0 * sw2 : 0;
    };
    if (wave < nsteps) {
      bf16x8 cur[NB], nxt[NB];
      uint32_t off;
      int valid;
      locate(wave, off, valid);
      load_frags(cur, off, valid);
      for (int st = wave; st < nsteps; st += kPbWaves) {
        const bool more = st + kPbWaves < nsteps;
        if (more) {                                // the next step's operands are read before this step's products
          locate(st + kPbWaves, off, valid);
          load_frags(nxt, off, valid);
        }
        int t = 0;
#pragma unroll
        for (int bi = 0; bi < NB; ++bi)
#pragma unroll
          for (int bj = 0; bj <= bi; ++bj, ++t) acc[t] = mfma_bf16(cur[bi], cur[bj], acc[t]);
        if (more) {
#pragma unroll
          for (int b = 0; b < NB; ++b) cur[b] = nxt[b];
        }
      }
    }
  }
  // The four waves' tiles are summed through the LDS in a fixed order, ((w3 + w2) + w1) + w0: a wave writes its tiles,
  // the next one adds them to its own (write-only and read-only passes, so the LDS accesses of a pass are in flight
  // together), and wave 0 stores the work group's partial.
  float* const red = reinterpret_cast<float*>(pb_smem);
  __syncthreads();
  for (int w = kPbWaves - 1; w > 0; --w) {
    if (wave == w) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) red[(t * 16 + e) * 64 + lane] = acc[t][e];
    }
    __syncthreads();
    if (wave == w - 1) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] += red[(t * 16 + e) * 64 + lane];
        __builtin_amdgcn_sched_barrier(0);          // a tile at a time: the reads of all tiles at once would not fit the registers
      }
    }
    __syncthreads();
  }
  if (wave == 0) {
    float* __restrict__ out = p.ws + static_cast<int64_t>(blockIdx.x) * NT * 1024;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) out[(t * 16 + e) * 64 + lane] = acc[t][e];
  }
}

// Sums the work groups' partials: a block takes 32 groups of four neighbouring tile elements, its 8 thread rows a
// slice of the partials each; the slices are added in a fixed order, then alpha / beta and the mirror image.
static __global__ __launch_bounds__(256) void conv_patch_bf16_reduce_kernel(PatchParams p) {
  __shared__ floatx4 part[8][32];
  const int q = blockIdx.x * 32 + (threadIdx.x & 31), slice = threadIdx.x >> 5;
  const floatx4* __restrict__ w = reinterpret_cast<const floatx4*>(p.ws) + q;
  const int64_t step = static_cast<int64_t>(p.ntiles) * 256;
  floatx4 s[4] = {floatx4{}, floatx4{}, floatx4{}, floatx4{}};
  int g = slice;
  for (; g + 24 < p.nwg; g += 32) {
    s[0] += w[(g + 0) * step];
    s[1] += w[(g + 8) * step];
    s[2] += w[(g + 16) * step];
    s[3] += w[(g + 24) * step];
  }
  for (; g < p.nwg; g += 8) s[0] += w[g * step];
  part[slice][threadIdx.x & 31] = (s[0] + s[1]) + (s[2] + s[3]);
  __syncthreads();
  if (slice != 0) return;
  floatx4 sum = part[0][threadIdx.x];
#pragma unroll
  for (int k = 1; k < 8; ++k) sum += part[k][threadIdx.x];
  const int t = q >> 8, el = (q & 255) * 4;            // tile; reg * 64 + lane of the first of the four elements
  int bi, bj;
  patch_tile_blocks(t, bi, bj);
  const int reg = el >> 6, lane = el & 63;
  const int i = 32 * bi + 8 * (reg >> 2) + 4 * (lane >> 5) + (reg & 3);
  if (i >= p.d) return;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int j = 32 * bj + (lane & 31) + k;
    if (j >= p.d || (bi == bj && j > i)) continue;
    float v = p.alpha * sum[k];
    float* dst = p.A + static_cast<int64_t>(i) * p.lda + j;
    if (p.beta != 0.f) v += p.beta * *dst;
    *dst = v;
    if (i != j) p.A[static_cast<int64_t>(j) * p.lda + i] = v;
  }
}

// Fills the plan; false when the layer is not one for this kernel.
static bool conv_patch_plan(PatchParams& p, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                     int pw) {
  const int64_t d = C * kh * kw;
  if (d > kPatchMaxD || kh * kw == 1 || N > (1 << 20) || H > (1 << 15) || W > (1 << 15)) return false;
  if (C * H * W >= (1ll << 31)) return false;           // offsets inside an image are 32-bit
  const int64_t Ho = (H + 2 * ph - kh) / sh + 1, Wo = (W + 2 * pw - kw) / sw + 1;
  if (Ho <= 0 || Wo <= 0) return false;
  const int64_t PC = (Wo - 1) * sw + kw;
  const int64_t RS = PC | 1;
  int R = 0;
  for (int r = 8; r >= 1; --r) {
    const int64_t PR = static_cast<int64_t>(r - 1) * sh + kh;
    if ((C * PR * RS + 1) * 4 <= static_cast<int64_t>(kPatchMaxLds)) { R = r; break; }
  }
  if (R == 0) return false;
  if (R > Ho) R = static_cast<int>(Ho);
  p.N = static_cast<int>(N); p.C = static_cast<int>(C); p.H = static_cast<int>(H); p.W = static_cast<int>(W);
  p.kh = kh; p.kw = kw; p.strh = sh; p.strw = sw; p.ph = ph; p.pw = pw;
  p.Ho = static_cast<int>(Ho); p.Wo = static_cast<int>(Wo);
  p.R = R;
  p.strips_per_image = static_cast<int>((Ho + R - 1) / R);
  const int64_t total = N * p.strips_per_image;
  if (total > (1 << 30)) return false;
  p.total_strips = static_cast<int>(total);
  p.PR = (R - 1) * sh + kh; p.PC = static_cast<int>(PC); p.RS = static_cast<int>(RS); p.plane = p.PR * p.RS;
  p.d = static_cast<int>(d);
  p.nb = (p.d + 31) / 32;
  p.ntiles = p.nb * (p.nb + 1) / 2;
  p.tpw = p.ntiles > kPatchWaves ? 2 : 1;
  const int groups = (p.ntiles + p.tpw - 1) / p.tpw;
  p.KS = kPatchWaves / groups;
  p.mKK = make_magic(kh * kw); p.mKw = make_magic(kw); p.mPC = make_magic(p.PC); p.mC = make_magic(p.C);
  p.mPRPC = make_magic(p.PR);
  p.nwg = static_cast<int>(total < 512 ? total : 512);
  return true;
}

// The plan of the bf16 kernel for a layer conv_patch_plan() accepts (its window limit, in elements, is the wider
// one): the strip height that minimises rounds of work groups x (matrix steps + window staging) per strip.
static void conv_patch_bf16_plan(PatchParams& p) {
  constexpr int kCUs = 256;
  const int64_t PC = p.PC;
  p.G = (p.Wo + 7) / 8;
  p.mG = make_magic(p.G);
  p.L = p.chan_inner ? p.PC * p.C : p.PC;
  p.mL = make_magic(p.L);
  p.RSb = p.L | 1;
  p.tap_x = p.chan_inner ? p.C : 1;
  p.lead = p.pw * p.tap_x;
  p.Lvalid = p.W * p.tap_x;
  const int64_t RS = p.RSb, rows_per = p.chan_inner ? 1 : p.C;
  int best_r = p.R;                         // the fp32 kernel's strip height fits in any case
  double best = 1e300;
  for (int r = 1; r <= p.Ho && r <= 64; ++r) {
    const int64_t PR = static_cast<int64_t>(r - 1) * p.strh + p.kh;
    if (rows_per * PR * RS > kPbMaxWindow) break;
    const int64_t strips = static_cast<int64_t>(p.N) * ((p.Ho + r - 1) / r);
    if (strips > (1 << 30)) continue;
    const int64_t rounds = (strips + kCUs - 1) / kCUs;
    const int64_t steps = ((static_cast<int64_t>(r) * p.G + 1) / 2 + kPbWaves - 1) / kPbWaves;
    const double cost = static_cast<double>(rounds) * (500.0 * steps + 24.0 * ((p.C * PR * PC + kPbThreads - 1) / kPbThreads) + 1500.0);
    if (cost < best) { best = cost; best_r = r; }
  }
  p.R = best_r;
  p.strips_per_image = (p.Ho + p.R - 1) / p.R;
  p.total_strips = p.N * p.strips_per_image;
  p.PR = (p.R - 1) * p.strh + p.kh;
  p.mPRPC = make_magic(p.PR);
  p.Q = p.chan_inner ? p.PR : p.C * p.PR;
  p.tap_c = p.chan_inner ? 1 : p.PR * p.RSb;
  p.nwg = p.total_strips < kCUs ? p.total_strips : kCUs;
}

size_t conv_patch_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw) {
  PatchParams p;
  if (!conv_patch_plan(p, N, C, H, W, kh, kw, sh, sw, ph, pw)) return 0;
  const size_t f32 = static_cast<size_t>(p.nwg) * kPatchWaves * 2 * 1024 * sizeof(float);
  const size_t b16 = static_cast<size_t>(256) * p.ntiles * 1024 * sizeof(float);     // at most one partial per CU
  return f32 > b16 ? f32 : b16;            // whichever kernel the dtype of the call selects
}

template <typename T, int NB>
static void conv_patch_bf16_launch_nb(const PatchParams& p, hipStream_t stream) {
  size_t lds = static_cast<size_t>(p.Q) * p.RSb * 2 + 2;
  const size_t red = static_cast<size_t>(p.ntiles) * 1024 * sizeof(float);
  if (red > lds) lds = red;
  if (p.chan_inner) hipLaunchKernelGGL((conv_patch_bf16_kernel<T, NB, true>), dim3(p.nwg), dim3(kPbThreads), lds, stream, p);
  else hipLaunchKernelGGL((conv_patch_bf16_kernel<T, NB, false>), dim3(p.nwg), dim3(kPbThreads), lds, stream, p);
}

template <typename T>
static int conv_patch_bf16_launch(PatchParams& p, hipStream_t stream) {
  conv_patch_bf16_plan(p);
  switch (p.nb) {
    case 1: conv_patch_bf16_launch_nb<T, 1>(p, stream); break;
    case 2: conv_patch_bf16_launch_nb<T, 2>(p, stream); break;
    case 3: conv_patch_bf16_launch_nb<T, 3>(p, stream); break;
    case 4: conv_patch_bf16_launch_nb<T, 4>(p, stream); break;
    default: conv_patch_bf16_launch_nb<T, 5>(p, stream); break;
  }
  hipLaunchKernelGGL(conv_patch_bf16_reduce_kernel, dim3(p.ntiles * 8), dim3(256), 0, stream, p);
  return check_launch();
}

template <typename T>
static int conv_patch_launch(PatchParams& p, hipStream_t stream) {
  const size_t lds = (static_cast<size_t>(p.C) * p.plane + 1) * sizeof(float);
  if (p.tpw > 1) hipLaunchKernelGGL((conv_patch_syrk_kernel<T, true>), dim3(p.nwg), dim3(kPatchThreads), lds, stream, p);
  else hipLaunchKernelGGL((conv_patch_syrk_kernel<T, false>), dim3(p.nwg), dim3(kPatchThreads), lds, stream, p);
  hipLaunchKernelGGL(conv_patch_reduce_kernel, dim3(p.ntiles * 4), dim3(256), 0, stream, p);
  return check_launch();
}

int conv_patch_syrk(const void* x, int dtype, int64_t sn, int64_t sc, int64_t sh_el, int64_t sw_el, int64_t N, int64_t C,
                    int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw, float alpha, float beta,
                    float* A, int64_t lda, void* ws, size_t ws_bytes, hipStream_t stream) {
  PatchParams p;
  if (!conv_patch_plan(p, N, C, H, W, kh, kw, sh, sw, ph, pw)) return AK_ERR_UNSUPPORTED;
  if (lda < p.d) return AK_ERR_ARG;
  if (ws == nullptr || ws_bytes < conv_patch_ws_bytes(N, C, H, W, kh, kw, sh, sw, ph, pw)) return AK_ERR_WORKSPACE;
  p.x = x; p.sn = sn; p.sc = sc; p.sh = sh_el; p.sw = sw_el;
  p.chan_inner = (sc == 1 && sw_el == C && C > 1) ? 1 : 0;
  p.ws = static_cast<float*>(ws);
  p.alpha = alpha; p.beta = beta; p.A = A; p.lda = lda;
  if (dtype == AK_BF16) return conv_patch_bf16_launch<uint16_t>(p, stream);
  if (dtype == AK_F32_AS_BF16) return conv_patch_bf16_launch<float>(p, stream);
  return conv_patch_launch<float>(p, stream);
}

}  // namespace ak
