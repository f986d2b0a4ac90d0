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
struct Counters {
  int* ptr = nullptr;
  size_t count = 0;
};
// The calling thread's scratch buffers, one per stream it has launched on.  They belong to
// the thread: released when it ends (and by mcReleaseScratch), so a thread that runs one
// net and exits leaves no device memory behind.
struct ThreadScratch {
  std::vector<std::pair<hipStream_t, Workspace>> workspaces;
  std::vector<std::pair<hipStream_t, Counters>> counters;
  void release() {
    // hipFree waits for the device: no kernel still reads what is freed
    for (auto& e : workspaces)
      if (e.second.ptr) (void)hipFree(e.second.ptr);
    for (auto& e : counters)
      if (e.second.ptr) (void)hipFree(e.second.ptr);
    workspaces.clear();
    counters.clear();
  }
  ~ThreadScratch() { release(); }
};
thread_local ThreadScratch g_scratch;
}  // namespace

int stream_counters(hipStream_t st, size_t count, int** out) {
  Counters* c = nullptr;
  for (auto& e : g_scratch.counters)
    if (e.first == st) c = &e.second;
  if (!c) {
    g_scratch.counters.emplace_back(st, Counters());
    c = &g_scratch.counters.back().second;
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

int stream_workspace(hipStream_t st, size_t bytes, float** out) {
  Workspace* ws = nullptr;
  for (auto& e : g_scratch.workspaces)
    if (e.first == st) ws = &e.second;
  if (!ws) {
    g_scratch.workspaces.emplace_back(st, Workspace());
    ws = &g_scratch.workspaces.back().second;
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

extern "C" int mcReleaseScratch(void) {
  mchip::g_scratch.release();
  return 0;
}
