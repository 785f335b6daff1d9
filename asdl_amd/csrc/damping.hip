// pi-damping split and all-zero test for a batch of Kronecker factor pairs, on the device.
//   pass 1 (one work group per pair): traces of A and B, pi, lamA, lamB; a factor whose diagonal
//           has a non-zero entry is flagged non-zero straight away.
//   pass 2 (grid over row chunks): only for factors whose diagonal is entirely zero, scans the
//           whole matrix for a non-zero entry (exactly `not torch.all(X == 0)`).
#include "common.hpp"

namespace ak {

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  const int wave = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

static __global__ __launch_bounds__(256) void damping_trace_kernel(const float* const* A_list, const float* const* B_list,
                                                                   const int64_t* dims, float damping, float eps,
                                                                   float* lam_out, int* nonzero_out) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  float tr[2];
  int nz[2];
  for (int f = 0; f < 2; ++f) {
    const float* M = f == 0 ? A_list[b] : B_list[b];
    const int64_t d = dims[2 * b + f];
    float s = 0.f;
    int any = 0;
    for (int64_t i = threadIdx.x; i < d; i += 256) {
      const float v = M[i * d + i];
      s += v;
      any |= (v != 0.f);
    }
    tr[f] = block_sum(s, red);
    nz[f] = __syncthreads_or(any);
  }
  if (threadIdx.x == 0) {
    const float dA = static_cast<float>(dims[2 * b]), dB = static_cast<float>(dims[2 * b + 1]);
    const float pi = sqrtf((tr[0] / dA) / (tr[1] / dB));
    float lamA = damping, lamB = damping;
    if (pi != 0.f && pi != INFINITY) {   // NaN passes both tests, like the reference's Python comparison
      const float r = sqrtf(damping);
      const float ra = r * pi, rb = r / pi;
      lamA = (eps > ra) ? eps : ra;     // Python max(ra, eps): keeps ra when it is NaN
      lamB = (eps > rb) ? eps : rb;
    }
    lam_out[2 * b] = lamA;
    lam_out[2 * b + 1] = lamB;
    nonzero_out[2 * b] = nz[0] ? 1 : 0;
    nonzero_out[2 * b + 1] = nz[1] ? 1 : 0;
  }
}

// grid (chunks, 2, batch)
static __global__ __launch_bounds__(256) void damping_scan_kernel(const float* const* A_list, const float* const* B_list,
                                                                  const int64_t* dims, int* nonzero_out) {
  const int b = blockIdx.z, f = blockIdx.y;
  if (nonzero_out[2 * b + f] != 0) return;
  const float* M = f == 0 ? A_list[b] : B_list[b];
  const int64_t d = dims[2 * b + f];
  const int64_t total = d * d;
  int any = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256)
    any |= (M[i] != 0.f);
  if (__syncthreads_or(any) && threadIdx.x == 0) atomicOr(&nonzero_out[2 * b + f], 1);
}

// The same with factors that may be kept as n x d matrices of per-sample rows (rows > 0): their eigenvalue mean is
// sum(x^2) / d and their all-zero test is exact in this pass.  dims: [batch][4] = rows_A, d_A, rows_B, d_B;
// eig_scale (may be null): [batch][2] factors applied to the eigenvalue means.
static __global__ __launch_bounds__(256) void damping_trace_swift_kernel(const float* const* A_list,
                                                                         const float* const* B_list, const int64_t* dims,
                                                                         const float* eig_scale, float damping, float eps,
                                                                         float* lam_out, int* nonzero_out) {
  __shared__ float red[4];
  const int b = blockIdx.x;
  float mean[2];
  int nz[2];
  for (int f = 0; f < 2; ++f) {
    const float* M = f == 0 ? A_list[b] : B_list[b];
    const int64_t rows = dims[4 * b + 2 * f], d = dims[4 * b + 2 * f + 1];
    float s = 0.f;
    int any = 0;
    if (rows == 0) {
      for (int64_t i = threadIdx.x; i < d; i += 256) {
        const float v = M[i * d + i];
        s += v;
        any |= (v != 0.f);
      }
    } else {
      for (int64_t i = threadIdx.x; i < rows * d; i += 256) {
        const float v = M[i];
        s += v * v;
        any |= (v != 0.f);
      }
    }
    mean[f] = block_sum(s, red) / static_cast<float>(d) * (eig_scale != nullptr ? eig_scale[2 * b + f] : 1.f);
    nz[f] = __syncthreads_or(any);
  }
  if (threadIdx.x == 0) {
    const float pi = sqrtf(mean[0] / mean[1]);
    float lamA = damping, lamB = damping;
    if (pi != 0.f && pi != INFINITY) {
      const float r = sqrtf(damping);
      const float ra = r * pi, rb = r / pi;
      lamA = (eps > ra) ? eps : ra;
      lamB = (eps > rb) ? eps : rb;
    }
    lam_out[2 * b] = lamA;
    lam_out[2 * b + 1] = lamB;
    nonzero_out[2 * b] = nz[0] ? 1 : 0;
    nonzero_out[2 * b + 1] = nz[1] ? 1 : 0;
  }
}

// grid (chunks, 2, batch): square factors with an all-zero diagonal only
static __global__ __launch_bounds__(256) void damping_scan_swift_kernel(const float* const* A_list,
                                                                        const float* const* B_list, const int64_t* dims,
                                                                        int* nonzero_out) {
  const int b = blockIdx.z, f = blockIdx.y;
  if (nonzero_out[2 * b + f] != 0 || dims[4 * b + 2 * f] != 0) return;
  const float* M = f == 0 ? A_list[b] : B_list[b];
  const int64_t d = dims[4 * b + 2 * f + 1];
  const int64_t total = d * d;
  int any = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256)
    any |= (M[i] != 0.f);
  if (__syncthreads_or(any) && threadIdx.x == 0) atomicOr(&nonzero_out[2 * b + f], 1);
}

// Identity into the matrices whose factor was all zero (flag 0); the others are left alone.
__global__ __launch_bounds__(256) void identity_where_zero_kernel(float* const* __restrict__ out_list,
                                                                   const int64_t* __restrict__ dims,
                                                                   const int* __restrict__ nonzero,
                                                                   const int64_t* __restrict__ flag_index) {
  const int m = blockIdx.y;
  if (nonzero[flag_index[m]] != 0) return;
  const int64_t d = dims[m], total = d * d;
  float* __restrict__ out = out_list[m];
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * 256)
    out[i] = (i / d == i % d) ? 1.f : 0.f;
}

}  // namespace ak

extern "C" int ak_identity_where_zero(float* const* out_list, const int64_t* dims, const int* nonzero,
                                      const int64_t* flag_index, int count, ak_stream_t stream) {
  if (out_list == nullptr || dims == nullptr || nonzero == nullptr || flag_index == nullptr || count <= 0)
    return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::identity_where_zero_kernel, dim3(32, count), dim3(256), 0, static_cast<hipStream_t>(stream),
                     out_list, dims, nonzero, flag_index);
  return ak::check_launch();
}

extern "C" int ak_kron_damping_swift(const float* const* A_list, const float* const* B_list, const int64_t* dims,
                                     const float* eig_scale, int batch, float damping, float eps, float* lam_out,
                                     int* nonzero_out, ak_stream_t stream) {
  if (A_list == nullptr || B_list == nullptr || dims == nullptr || lam_out == nullptr || nonzero_out == nullptr ||
      batch <= 0)
    return AK_ERR_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(ak::damping_trace_swift_kernel, dim3(batch), dim3(256), 0, s, A_list, B_list, dims, eig_scale,
                     damping, eps, lam_out, nonzero_out);
  hipLaunchKernelGGL(ak::damping_scan_swift_kernel, dim3(64, 2, batch), dim3(256), 0, s, A_list, B_list, dims,
                     nonzero_out);
  return ak::check_launch();
}

extern "C" int ak_kron_damping(const float* const* A_list, const float* const* B_list, const int64_t* dims, int batch,
                               float damping, float eps, float* lam_out, int* nonzero_out, ak_stream_t stream) {
  if (A_list == nullptr || B_list == nullptr || dims == nullptr || lam_out == nullptr || nonzero_out == nullptr ||
      batch <= 0)
    return AK_ERR_ARG;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(ak::damping_trace_kernel, dim3(batch), dim3(256), 0, s, A_list, B_list, dims, damping, eps,
                     lam_out, nonzero_out);
  hipLaunchKernelGGL(ak::damping_scan_kernel, dim3(64, 2, batch), dim3(256), 0, s, A_list, B_list, dims, nonzero_out);
  return ak::check_launch();
}
