// Status text, version and the optional per-kernel timing hook of the C ABI.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/gs_hip.h"

namespace gs {
namespace {
thread_local char g_error_text[512] = "";

// profiling state: a ring of event pairs for the one enabled launch site
std::atomic<bool> g_profile_on{false};
char g_profile_name[64] = "";
std::mutex g_profile_mu;
std::vector<hipEvent_t> g_start, g_stop;
int g_used = 0;
int g_stride = 1;     // time every g_stride-th launch of the site
int g_seen = 0;       // launches of the site since enable
constexpr int kMaxPairs = 4096;
}  // namespace

void set_error_text(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error_text, sizeof(g_error_text), fmt, ap);
  va_end(ap);
}

void profile_begin(const char* name, hipStream_t stream, int* slot) {
  *slot = -1;
  if (!g_profile_on.load(std::memory_order_relaxed)) return;
  std::lock_guard<std::mutex> lock(g_profile_mu);
  if (std::strcmp(name, g_profile_name) != 0 || g_used >= kMaxPairs) return;
  if (g_seen++ % g_stride != 0) return;
  if (g_used == static_cast<int>(g_start.size())) {
    hipEvent_t a, b;
    if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return;
    g_start.push_back(a);
    g_stop.push_back(b);
  }
  *slot = g_used++;
  (void)hipEventRecord(g_start[*slot], stream);
}

void profile_end(hipStream_t stream, int slot) {
  std::lock_guard<std::mutex> lock(g_profile_mu);
  (void)hipEventRecord(g_stop[slot], stream);
}
}  // namespace gs

extern "C" {

const char* gs_status_string(int status) {
  switch (status) {
    case GS_OK:
      return "ok";
    case GS_ERR_INVALID_ARG:
    case GS_ERR_WORKSPACE:
    case GS_ERR_UNSUPPORTED:
    case GS_ERR_LAUNCH:
      return gs::g_error_text[0] ? gs::g_error_text : "error (no detail recorded)";
    default:
      return "unknown status";
  }
}

int gs_version(void) { return 100; }

int gs_profile_stride(int every) {
  std::lock_guard<std::mutex> lock(gs::g_profile_mu);
  gs::g_stride = every < 1 ? 1 : every;
  return GS_OK;
}

int gs_profile_enable(const char* launch_site) {
  std::lock_guard<std::mutex> lock(gs::g_profile_mu);
  gs::g_used = 0;
  gs::g_seen = 0;
  if (!launch_site || !launch_site[0]) {
    gs::g_profile_on.store(false);
    gs::g_profile_name[0] = 0;
    return GS_OK;
  }
  std::snprintf(gs::g_profile_name, sizeof(gs::g_profile_name), "%s", launch_site);
  gs::g_profile_on.store(true);
  return GS_OK;
}

int gs_profile_collect(double* total_ms, int64_t* launches, double* per_launch_ms, int64_t cap) {
  std::lock_guard<std::mutex> lock(gs::g_profile_mu);
  double total = 0.0;
  for (int i = 0; i < gs::g_used; ++i) {
    if (hipEventSynchronize(gs::g_stop[i]) != hipSuccess) return GS_ERR_LAUNCH;
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, gs::g_start[i], gs::g_stop[i]) != hipSuccess) return GS_ERR_LAUNCH;
    total += ms;
    if (per_launch_ms && i < cap) per_launch_ms[i] = ms;
  }
  if (total_ms) *total_ms = total;
  if (launches) *launches = gs::g_used;
  gs::g_used = 0;
  return GS_OK;
}

}  // extern "C"
