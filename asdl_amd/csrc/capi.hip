// Version and error strings of the C ABI.
#include "common.hpp"

extern "C" int ak_version(void) { return 100; }

extern "C" const char* ak_error_string(int code) {
  switch (code) {
    case AK_OK: return "ok";
    case AK_ERR_ARG: return "bad argument (null pointer, negative size, leading dimension too small or unknown dtype)";
    case AK_ERR_WORKSPACE: return "workspace missing or smaller than the matching *_ws_bytes() query";
    case AK_ERR_UNSUPPORTED: return "configuration not supported by this kernel";
    case AK_ERR_LAUNCH: return "HIP reported a kernel launch failure";
    default: return "unknown error code";
  }
}

namespace ak {
static __global__ __launch_bounds__(256) void debug_copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                                int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
    dst[i] = src[i];
}
}  // namespace ak

// Measurement hook, not part of the interface: a plain copy of `bytes` bytes (multiple of 16), i.e. exactly `bytes`
// read from and `bytes` written to device memory, against which hardware traffic counters are calibrated.
extern "C" int ak_debug_copy(const void* src, void* dst, int64_t bytes, ak_stream_t stream) {
  if (src == nullptr || dst == nullptr || bytes <= 0 || bytes % 16 != 0) return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::debug_copy_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float4*>(src), static_cast<float4*>(dst), bytes / 16);
  return ak::check_launch();
}
