// Per-thread device context, pooled allocator and the host/device mirror.
//
// Replaces the CUDA side of the reference's src/common.{hpp,cpp} (thread-local
// Caffe singleton: mode, device) and src/syncedmem.{hpp,cpp} (SyncedMemory with
// a 4-state head + thread-local MemoryPool) with a HIP design: one stream per
// thread, pinned host blocks from hipHostMalloc, device blocks from hipMalloc,
// hipMemcpyAsync on that stream, and a stream synchronisation only where a
// host pointer is handed out.
#ifndef MCHIP_RUNTIME_DEVICE_HPP_
#define MCHIP_RUNTIME_DEVICE_HPP_

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <memory>
#include <mutex>

#include "caffe/base.hpp"

#define HIP_CHECK(expr)                                                                   \
  do {                                                                                    \
    hipError_t hip_check_e_ = (expr);                                                     \
    CHECK(hip_check_e_ == hipSuccess) << #expr << ": " << hipGetErrorString(hip_check_e_); \
  } while (0)

// Kernel-level entry points report through a return code + mcLastError().
#define MC_CHECK(expr) CHECK((expr) == 0) << mcLastError()

namespace caffe {

class MemoryPool;

// What the reference keeps in its thread-local `Caffe` object
// (reference src/common.hpp:75-116, common.cpp:7-148).
class Context {
 public:
  static Context& Get();
  static DeviceMode mode() { return Get().mode_; }
  static bool gpu_available();

  void SetMode(DeviceMode mode, int device);
  int device() const { return device_; }
  // The thread's stream; created on first use in GPU mode.
  hipStream_t stream();
  // Waits for everything queued on the stream.
  void Sync();
  // Incremented by every Sync(); lets owners of host buffers know whether an
  // asynchronous copy they queued can still be in flight.
  uint64_t sync_epoch() const { return sync_epoch_; }
  const std::shared_ptr<MemoryPool>& pool() { return pool_; }
  ~Context();

 private:
  Context();
  DeviceMode mode_;
  int device_;
  hipStream_t stream_;
  bool stream_ready_;
  uint64_t sync_epoch_;
  std::shared_ptr<MemoryPool> pool_;
};

// Size-keyed free lists of host (pinned when a device exists) and device
// blocks.  A request is served by the smallest free block that is large enough
// and at most twice the request; otherwise a new block is allocated
// (reference syncedmem.cpp:177-347 uses the same "has/2 <= wants" rule).
class MemoryPool {
 public:
  struct Block {
    void* ptr = nullptr;
    size_t size = 0;
    int device = -1;     // -1: host
    bool pinned = false;
  };
  ~MemoryPool();
  Block RequestHost(size_t size);
  Block RequestDevice(size_t size, int device);
  void Return(const Block& b);
  void Clear();
  MemPoolState64 GetState();

 private:
  std::mutex mu_;
  std::multimap<size_t, Block> free_host_;
  std::multimap<std::pair<int, size_t>, Block> free_dev_;
  long long host_total_ = 0, dev_total_ = 0, host_unused_ = 0, dev_unused_ = 0;
};

class SyncedMemory {
 public:
  enum SyncedHead { UNINITIALIZED, HEAD_AT_CPU, HEAD_AT_GPU, SYNCED };
  explicit SyncedMemory(size_t size);
  ~SyncedMemory();
  const void* cpu_data();
  void* mutable_cpu_data();
  const void* gpu_data();
  void* mutable_gpu_data();
  SyncedHead head() const { return head_; }
  size_t size() const { return size_; }
  // Bumped by every mutable_* access: cheap "did the contents possibly change".
  uint64_t version() const { return version_; }

 private:
  void to_cpu();
  void to_gpu();
  void wait_pending_h2d();
  size_t size_;
  SyncedHead head_;
  MemoryPool::Block host_, dev_;
  std::shared_ptr<MemoryPool> pool_;
  uint64_t version_;
  uint64_t h2d_epoch_;   // sync epoch at which an async H2D was queued
  bool h2d_pending_;
  DISABLE_COPY_AND_ASSIGN(SyncedMemory);
};

}  // namespace caffe

#endif  // MCHIP_RUNTIME_DEVICE_HPP_
