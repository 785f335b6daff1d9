// Conv2d input factor for layers with few input channels (d = C*kh*kw <= 160, e.g. the 3-channel 7x7 stem of
// a ResNet): A = sum over output positions of p p^T, p the (c,ky,kx)-ordered patch, in fp32.
//
// The unfolded matrix has d short rows per position and would be gathered element by element; instead each work
// group stages the input window of a strip of R output rows of one image in LDS once ([c][row][col] planes, zero
// padding materialised) and the lanes of the fp32 matrix instruction read their patch element straight from that
// window: lane l of v_mfma_f32_32x32x2_f32 supplies patch element (32*block + l%32) of position (2*step + l/32).
// The lower 32 x 32 tiles of the (padded) d x d result are spread over the 8 waves; a work group walks over
// several strips and writes one partial per wave and tile slot, summed by a second kernel that also applies
// alpha / beta and mirrors the result.  Input: fp32 or bf16 with arbitrary element strides (NCHW and NHWC alike).
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
  float* ws;                     // [grid][wave][slot][16][64]
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

// Fills the plan; false when the layer is not one for this kernel.
static bool conv_patch_plan(PatchParams& p, int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph,
                     int pw) {
  const int64_t d = C * kh * kw;
  if (d > kPatchMaxD || kh * kw == 1 || N > (1 << 20) || H > (1 << 15) || W > (1 << 15)) return false;
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

size_t conv_patch_ws_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int kh, int kw, int sh, int sw, int ph, int pw) {
  PatchParams p;
  if (!conv_patch_plan(p, N, C, H, W, kh, kw, sh, sw, ph, pw)) return 0;
  return static_cast<size_t>(p.nwg) * kPatchWaves * 2 * 1024 * sizeof(float);
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
  if (ws == nullptr || ws_bytes < static_cast<size_t>(p.nwg) * kPatchWaves * 2 * 1024 * sizeof(float))
    return AK_ERR_WORKSPACE;
  p.x = x; p.sn = sn; p.sc = sc; p.sh = sh_el; p.sw = sw_el;
  p.chan_inner = (sc == 1 && C > 1) ? 1 : 0;
  p.ws = static_cast<float*>(ws);
  p.alpha = alpha; p.beta = beta; p.A = A; p.lda = lda;
  return dtype == AK_BF16 ? conv_patch_launch<uint16_t>(p, stream) : conv_patch_launch<float>(p, stream);
}

}  // namespace ak
