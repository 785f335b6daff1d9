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
