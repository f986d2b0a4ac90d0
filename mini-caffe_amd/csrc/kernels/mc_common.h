// Shared helpers for the device kernels: error capture and launch geometry.
#ifndef MCHIP_COMMON_H_
#define MCHIP_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <string>

namespace mchip {

// Thread-local message returned by mcLastError().
std::string& last_error();

inline int fail(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error() = buf;
  return -1;
}

#define MC_HIP(expr)                                                        \
  do {                                                                      \
    hipError_t e_ = (expr);                                                 \
    if (e_ != hipSuccess)                                                   \
      return ::mchip::fail("%s failed: %s (%s:%d)", #expr,                  \
                           hipGetErrorString(e_), __FILE__, __LINE__);      \
  } while (0)

#define MC_REQUIRE(cond, ...)                                               \
  do {                                                                      \
    if (!(cond)) return ::mchip::fail(__VA_ARGS__);                         \
  } while (0)

// Reports a failed launch (bad configuration shows up here, not at sync).
#define MC_LAUNCH_CHECK() MC_HIP(hipGetLastError())

constexpr int kWave = 64;            // CDNA wavefront width
constexpr int kNumXcd = 8;           // MI355X: 8 XCDs, each with its own L2
constexpr int kNumCu = 256;

inline int ceil_div(long a, long b) { return static_cast<int>((a + b - 1) / b); }

// Grid for a grid-stride elementwise kernel: enough blocks to cover n once,
// capped at a few waves per CU so tails stay short.
inline int ew_blocks(long n, int threads, int per_thread = 1) {
  long b = (n + static_cast<long>(threads) * per_thread - 1) /
           (static_cast<long>(threads) * per_thread);
  const long cap = static_cast<long>(kNumCu) * 16;
  if (b > cap) b = cap;
  if (b < 1) b = 1;
  return static_cast<int>(b);
}

// Device scratch for partial results that one call writes and reads back (the
// slices of a split-K contraction, per-part statistics): one grow-only buffer per
// (host thread, stream), owned by the thread: freed when the thread ends or calls
// mcReleaseScratch.  Work on one stream is ordered, so consecutive calls share it.
// Growing frees the old buffer, which waits for the device.
int stream_workspace(hipStream_t st, size_t bytes, float** out);

// Arrival counters for kernels whose workgroups hand work to the last one to
// finish: one grow-only array of ints per (host thread, stream), zero when it is
// handed out.  A kernel that counts in it leaves every counter at zero again.
int stream_counters(hipStream_t st, size_t count, int** out);

}  // namespace mchip

#endif  // MCHIP_COMMON_H_
