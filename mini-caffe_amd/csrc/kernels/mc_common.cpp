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
thread_local std::vector<std::pair<hipStream_t, Workspace>> g_workspaces;
}  // namespace

int stream_workspace(hipStream_t st, size_t bytes, float** out) {
  Workspace* ws = nullptr;
  for (auto& e : g_workspaces)
    if (e.first == st) ws = &e.second;
  if (!ws) {
    g_workspaces.emplace_back(st, Workspace());
    ws = &g_workspaces.back().second;
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
