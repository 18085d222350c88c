// Library-wide pieces of the C ABI: version, thread-local error string, launch-status check.
#include "common.hpp"

#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

namespace {
thread_local char g_error[512] = "";

bool g_timing = false;
std::mutex g_timing_mu;
std::map<std::string, std::vector<std::pair<hipEvent_t, hipEvent_t>>> g_timing_events;
}

MltsKernelTimer::MltsKernelTimer(const char* name, hipStream_t stream)
    : name_(name), stream_(stream), start_(nullptr), active_(g_timing) {
  if (!active_) return;
  if (hipEventCreate(&start_) != hipSuccess || hipEventRecord(start_, stream_) != hipSuccess) active_ = false;
}

MltsKernelTimer::~MltsKernelTimer() {
  if (!active_) return;
  hipEvent_t stop;
  if (hipEventCreate(&stop) != hipSuccess) return;
  if (hipEventRecord(stop, stream_) != hipSuccess) return;
  std::lock_guard<std::mutex> lock(g_timing_mu);
  g_timing_events[name_].emplace_back(start_, stop);
}

extern "C" void mlts_kernel_timing_enable(int enable) {
  std::lock_guard<std::mutex> lock(g_timing_mu);
  g_timing = enable != 0;
  for (auto& kv : g_timing_events)
    for (auto& ev : kv.second) {
      (void)hipEventDestroy(ev.first);
      (void)hipEventDestroy(ev.second);
    }
  g_timing_events.clear();
}

extern "C" int mlts_kernel_timing_read(const char* name, double* total_ms, int64_t* launches) {
  if (!name || !total_ms || !launches) {
    mlts_set_error("mlts_kernel_timing_read: null argument");
    return MLTS_ERR_INVALID;
  }
  std::lock_guard<std::mutex> lock(g_timing_mu);
  *total_ms = 0.0;
  *launches = 0;
  auto it = g_timing_events.find(name);
  if (it == g_timing_events.end()) return MLTS_OK;
  for (auto& ev : it->second) {
    if (hipEventSynchronize(ev.second) != hipSuccess) continue;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, ev.first, ev.second) == hipSuccess) {
      *total_ms += ms;
      *launches += 1;
    }
  }
  return MLTS_OK;
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

extern "C" int mlts_abi_version(void) { return 4; }
extern "C" const char* mlts_last_error(void) { return g_error; }
