// Opt-in kernel timing: while enabled, the decode entry points launch their dominant kernel with
// a pair of HIP events attached to the dispatch (launch.h: launch_timed), so a benchmark can read that
// kernel's duration without an external profiler.  Not for use under graph capture.
#include <vector>

#include "launch.h"

namespace xllm_mi355 {

namespace {
struct ProfileState {
  std::vector<hipEvent_t> start, stop;
  std::vector<char> skipped;
  int used = 0;
  bool enabled = false;
};
ProfileState g_profile;
}  // namespace

bool profile_events(hipEvent_t* start, hipEvent_t* stop) {
  ProfileState& p = g_profile;
  if (!p.enabled || p.used >= static_cast<int>(p.start.size())) return false;
  *start = p.start[p.used];
  *stop = p.stop[p.used];
  p.skipped[p.used] = 0;
  return true;
}

void profile_commit() { ++g_profile.used; }

void profile_skip() {
  ProfileState& p = g_profile;
  if (!p.enabled || p.used >= static_cast<int>(p.start.size())) return;
  p.skipped[p.used++] = 1;
}

}  // namespace xllm_mi355

using namespace xllm_mi355;

extern "C" {

int xllm_mi355_profile_enable(int capacity) {
  ProfileState& p = g_profile;
  if (capacity < 0) return XLLM_MI355_EINVAL;
  while (static_cast<int>(p.start.size()) < capacity) {
    hipEvent_t a, b;
    hipError_t e = hipEventCreate(&a);
    if (e != hipSuccess) return static_cast<int>(e);
    e = hipEventCreate(&b);
    if (e != hipSuccess) return static_cast<int>(e);
    p.start.push_back(a);
    p.stop.push_back(b);
  }
  p.skipped.assign(p.start.size(), 0);
  p.used = 0;
  p.enabled = capacity > 0;
  return XLLM_MI355_OK;
}

int xllm_mi355_profile_collect(float* ms_out, int max_n) {
  ProfileState& p = g_profile;
  p.enabled = false;
  int n = 0;
  for (; n < p.used && n < max_n; ++n) {
    if (p.skipped[n]) {
      ms_out[n] = 0.0f;
      continue;
    }
    hipError_t e = hipEventSynchronize(p.stop[n]);
    if (e != hipSuccess) return -static_cast<int>(e) - 1000;
    e = hipEventElapsedTime(&ms_out[n], p.start[n], p.stop[n]);
    if (e != hipSuccess) return -static_cast<int>(e) - 1000;
  }
  p.used = 0;
  return n;
}

}  // extern "C"
