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
    case AK_ERR_TOO_LARGE: return "sizes beyond the fixed maximum of this entry point's built-in scratch memory";
    default: return "unknown error code";
  }
}

namespace ak {
static __global__ __launch_bounds__(256) void copy_bytes_kernel(const float4* __restrict__ src, float4* __restrict__ dst,
                                                                int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
    dst[i] = src[i];
}
}  // namespace ak

// Measurement aid: a plain copy of `bytes` bytes (multiple of 16), i.e. exactly `bytes`
// read from and `bytes` written to device memory, against which hardware traffic counters are calibrated.
extern "C" int ak_copy_bytes(const void* src, void* dst, int64_t bytes, ak_stream_t stream) {
  if (src == nullptr || dst == nullptr || bytes <= 0 || bytes % 16 != 0) return AK_ERR_ARG;
  hipLaunchKernelGGL(ak::copy_bytes_kernel, dim3(4096), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const float4*>(src), static_cast<float4*>(dst), bytes / 16);
  return ak::check_launch();
}

// ---- stream helpers -------------------------------------------------------------------------------------------
// Thin wrappers over the HIP runtime this library is linked against, for hosts that run the statistics kernels on a
// side stream of their own: ordering a side stream after the producing stream costs two runtime calls here instead of
// the host framework's stream-context machinery.  Events are created by the caller and live until it destroys them.

extern "C" int ak_event_create(void** event, int timing) {
  if (event == nullptr) return AK_ERR_ARG;
  hipEvent_t ev;
  if (hipEventCreateWithFlags(&ev, timing ? hipEventDefault : hipEventDisableTiming) != hipSuccess) return AK_ERR_LAUNCH;
  *event = ev;
  return AK_OK;
}

extern "C" int ak_event_destroy(void* event) {
  if (event == nullptr) return AK_ERR_ARG;
  return hipEventDestroy(static_cast<hipEvent_t>(event)) == hipSuccess ? AK_OK : AK_ERR_LAUNCH;
}

extern "C" int ak_event_record(void* event, ak_stream_t stream) {
  if (event == nullptr) return AK_ERR_ARG;
  return hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)) == hipSuccess ? AK_OK
                                                                                                         : AK_ERR_LAUNCH;
}

// `after` waits for everything enqueued on `before` so far (event: scratch, re-recordable).
extern "C" int ak_stream_order(ak_stream_t before, ak_stream_t after, void* event) {
  if (event == nullptr) return AK_ERR_ARG;
  hipEvent_t ev = static_cast<hipEvent_t>(event);
  if (hipEventRecord(ev, static_cast<hipStream_t>(before)) != hipSuccess) return AK_ERR_LAUNCH;
  if (hipStreamWaitEvent(static_cast<hipStream_t>(after), ev, 0) != hipSuccess) return AK_ERR_LAUNCH;
  return AK_OK;
}

// Milliseconds between two recorded timing events; both must have completed.
extern "C" int ak_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (start == nullptr || stop == nullptr || ms == nullptr) return AK_ERR_ARG;
  return hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) == hipSuccess
             ? AK_OK
             : AK_ERR_LAUNCH;
}
