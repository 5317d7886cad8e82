// Host-side plumbing shared by every C-ABI entry point: status strings, the thread-local
// last-error message and the post-launch check.

#include <stdarg.h>
#include <stdio.h>

#include "device_common.hpp"

namespace areno {

namespace {
thread_local char g_last_error[512] = "";
}

void set_error(const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, args);
  va_end(args);
}

int fail(int status, const char* fmt, ...) {
  va_list args;
  va_start(args, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, args);
  va_end(args);
  return status;
}

int check_launch(const char* what) {
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail(ARENO_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(err));
  return ARENO_OK;
}

size_t dtype_size(int dtype) {
  switch (dtype) {
    case ARENO_DT_F32: return 4;
    case ARENO_DT_F16:
    case ARENO_DT_BF16: return 2;
    case ARENO_DT_I8:
    case ARENO_DT_FP8_E4M3: return 1;
    default: return 0;
  }
}

bool is_quantized(int dtype) { return dtype == ARENO_DT_I8 || dtype == ARENO_DT_FP8_E4M3; }

}  // namespace areno

extern "C" int areno_hip_abi_version(void) { return ARENO_HIP_ABI_VERSION; }

extern "C" const char* areno_hip_status_string(int status) {
  switch (status) {
    case ARENO_OK: return "ok";
    case ARENO_ERR_INVALID_ARGUMENT: return "invalid argument";
    case ARENO_ERR_UNSUPPORTED: return "unsupported dtype or shape";
    case ARENO_ERR_WORKSPACE: return "workspace missing or too small";
    case ARENO_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

extern "C" const char* areno_hip_last_error(void) { return areno::g_last_error; }
