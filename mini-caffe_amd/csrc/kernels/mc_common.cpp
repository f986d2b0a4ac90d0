#include "mc_common.h"
#include "mchip/kernels.h"

#include <utility>
#include <vector>

namespace mchip {
std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}

namespace {
struct Workspace {
  float* ptr = nullptr;
  size_t bytes = 0;
};
thread_local std::vector<std::pair<hipStream_t, Workspace>> g_workspaces[2];
struct Counters {
  int* ptr = nullptr;
  size_t count = 0;
};
thread_local std::vector<std::pair<hipStream_t, Counters>> g_counters;
}  // namespace

int stream_counters(hipStream_t st, size_t count, int** out) {
  Counters* c = nullptr;
  for (auto& e : g_counters)
    if (e.first == st) c = &e.second;
  if (!c) {
    g_counters.emplace_back(st, Counters());
    c = &g_counters.back().second;
  }
  if (c->count < count) {
    if (c->ptr) MC_HIP(hipFree(c->ptr));  // waits for the device: every user has put its zeros back
    c->ptr = nullptr;
    c->count = 0;
    count = (count + 4095) / 4096 * 4096;
    MC_HIP(hipMalloc(&c->ptr, count * sizeof(int)));
    MC_HIP(hipMemset(c->ptr, 0, count * sizeof(int)));
    MC_HIP(hipDeviceSynchronize());  // the zeros are in place before a kernel on any stream counts
    c->count = count;
  }
  *out = c->ptr;
  return 0;
}

int stream_workspace(hipStream_t st, size_t bytes, float** out, int slot) {
  Workspace* ws = nullptr;
  auto& all = g_workspaces[slot != 0];
  for (auto& e : all)
    if (e.first == st) ws = &e.second;
  if (!ws) {
    all.emplace_back(st, Workspace());
    ws = &all.back().second;
  }
  if (ws->bytes < bytes) {
    if (ws->ptr) MC_HIP(hipFree(ws->ptr));  // waits for the device
    ws->ptr = nullptr;
    ws->bytes = 0;
    MC_HIP(hipMalloc(&ws->ptr, bytes));
    ws->bytes = bytes;
  }
  *out = ws->ptr;
  return 0;
}
}  // namespace mchip

extern "C" const char* mcLastError(void) { return mchip::last_error().c_str(); }
