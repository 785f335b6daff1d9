// Lower-triangle packing of a symmetric matrix, row direction (the on-disk form of a saved factor):
//   tril[i*(i+1)/2 + j] = mat[i][j], j <= i          and back: mat[i][j] = mat[j][i] = tril[i*(i+1)/2 + j].
// Pure index work, bound by the HBM; one thread per matrix element of the square, so that the reads (pack) or
// the writes (unpack) of a row are coalesced.
#include "common.hpp"

namespace ak {

static __global__ __launch_bounds__(256) void tril_pack_kernel(const float* __restrict__ mat, int64_t d, int64_t ld,
                                                               float* __restrict__ tril) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t i = blockIdx.y;
  if (j <= i && j < d) tril[i * (i + 1) / 2 + j] = mat[i * ld + j];
}

static __global__ __launch_bounds__(256) void tril_unpack_kernel(const float* __restrict__ tril, int64_t d, int64_t ld,
                                                                 float* __restrict__ mat) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t i = blockIdx.y;
  if (j >= d) return;
  mat[i * ld + j] = j <= i ? tril[i * (i + 1) / 2 + j] : tril[j * (j + 1) / 2 + i];
}

}  // namespace ak

extern "C" int ak_tril_pack(const float* mat, int64_t d, int64_t ld, float* tril, ak_stream_t stream) {
  if (mat == nullptr || tril == nullptr || d <= 0 || ld < d || d > 65535) return AK_ERR_ARG;
  dim3 grid(static_cast<unsigned>((d + 255) / 256), static_cast<unsigned>(d));
  hipLaunchKernelGGL(ak::tril_pack_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), mat, d, ld, tril);
  return ak::check_launch();
}

extern "C" int ak_tril_unpack(const float* tril, int64_t d, float* mat, int64_t ld, ak_stream_t stream) {
  if (mat == nullptr || tril == nullptr || d <= 0 || ld < d || d > 65535) return AK_ERR_ARG;
  dim3 grid(static_cast<unsigned>((d + 255) / 256), static_cast<unsigned>(d));
  hipLaunchKernelGGL(ak::tril_unpack_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), tril, d, ld, mat);
  return ak::check_launch();
}
