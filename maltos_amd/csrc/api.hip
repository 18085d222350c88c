// Library-wide pieces of the C ABI: version, thread-local error string, launch-status check.
#include "common.hpp"

namespace {
thread_local char g_error[512] = "";
}

void mlts_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int mlts_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    mlts_set_error("%s: HIP launch failed: %s", what, hipGetErrorString(e));
    return MLTS_ERR_LAUNCH;
  }
  return MLTS_OK;
}

extern "C" int mlts_abi_version(void) { return 1; }
extern "C" const char* mlts_last_error(void) { return g_error; }
