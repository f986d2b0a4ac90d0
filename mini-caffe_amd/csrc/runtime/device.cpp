#include "device.hpp"

#include <climits>
#include <cstdlib>
#include <cstring>

#include "mchip/kernels.h"

namespace caffe {

// ---------------------------------------------------------------------------
// Context
// ---------------------------------------------------------------------------

Context& Context::Get() {
  static thread_local Context ctx;
  return ctx;
}

Context::Context()
    : mode_(CPU), device_(0), stream_(nullptr), stream_ready_(false), sync_epoch_(1),
      pool_(std::make_shared<MemoryPool>()) {}

Context::~Context() {
  if (stream_ready_) (void)hipStreamDestroy(stream_);
}

bool Context::gpu_available() {
  static const bool available = [] {
    int n = 0;
    return hipGetDeviceCount(&n) == hipSuccess && n > 0;
  }();
  return available;
}

void Context::SetMode(DeviceMode mode, int device) {
  if (mode == GPU) {
    CHECK(gpu_available()) << "SetMode(GPU): no HIP device is visible to this process";
    int n = 0;
    HIP_CHECK(hipGetDeviceCount(&n));
    CHECK(device >= 0 && device < n) << "SetMode(GPU): invalid device id " << device << " ("
                                     << n << " device(s) present)";
    if (stream_ready_ && device != device_) {
      Sync();
      HIP_CHECK(hipStreamDestroy(stream_));
      stream_ready_ = false;
    }
    HIP_CHECK(hipSetDevice(device));
    device_ = device;
  }
  mode_ = mode;
}

hipStream_t Context::stream() {
  if (!stream_ready_) {
    HIP_CHECK(hipSetDevice(device_));
    HIP_CHECK(hipStreamCreate(&stream_));  // default priority
    stream_ready_ = true;
  }
  return stream_;
}

void Context::Sync() {
  if (stream_ready_) HIP_CHECK(hipStreamSynchronize(stream_));
  ++sync_epoch_;
}

bool GPUAvailable() { return Context::gpu_available(); }

void SetMode(DeviceMode mode, int device) { Context::Get().SetMode(mode, device); }

MemPoolState64 MemPoolGetState64() { return Context::Get().pool()->GetState(); }

MemPoolState MemPoolGetState() {
  const MemPoolState64 s = MemPoolGetState64();
  auto sat = [](long long v) { return v > INT_MAX ? INT_MAX : static_cast<int>(v); };
  MemPoolState r;
  r.gpu_mem = sat(s.gpu_mem);
  r.cpu_mem = sat(s.cpu_mem);
  r.unused_gpu_mem = sat(s.unused_gpu_mem);
  r.unused_cpu_mem = sat(s.unused_cpu_mem);
  return r;
}

void MemPoolClear() {
  Context::Get().Sync();
  Context::Get().pool()->Clear();
  (void)mcReleaseScratch();  // the kernels' own scratch of this thread
}

// ---------------------------------------------------------------------------
// MemoryPool
// ---------------------------------------------------------------------------

namespace {
size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
}  // namespace

MemoryPool::~MemoryPool() { Clear(); }

MemoryPool::Block MemoryPool::RequestHost(size_t size) {
  size = round_up(size ? size : 1, 256);
  {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = free_host_.lower_bound(size);
    if (it != free_host_.end() && it->first <= 2 * size) {
      Block b = it->second;
      free_host_.erase(it);
      host_unused_ -= b.size;
      return b;
    }
  }
  Block b;
  b.size = size;
  b.device = -1;
  if (Context::gpu_available()) {
    // Pinned, so that hipMemcpyAsync is truly asynchronous.
    HIP_CHECK(hipHostMalloc(&b.ptr, size, hipHostMallocDefault));
    b.pinned = true;
  } else {
    b.ptr = std::aligned_alloc(256, size);
    CHECK(b.ptr) << "host allocation of " << size << " bytes failed";
  }
  std::lock_guard<std::mutex> lk(mu_);
  host_total_ += size;
  return b;
}

MemoryPool::Block MemoryPool::RequestDevice(size_t size, int device) {
  size = round_up(size ? size : 1, 256);
  {
    std::lock_guard<std::mutex> lk(mu_);
    auto it = free_dev_.lower_bound(std::make_pair(device, size));
    if (it != free_dev_.end() && it->first.first == device && it->first.second <= 2 * size) {
      Block b = it->second;
      free_dev_.erase(it);
      dev_unused_ -= b.size;
      return b;
    }
  }
  Block b;
  b.size = size;
  b.device = device;
  HIP_CHECK(hipSetDevice(device));
  hipError_t e = hipMalloc(&b.ptr, size);
  if (e != hipSuccess) {
    // Give cached blocks back and retry once before failing.
    (void)hipGetLastError();
    Clear();
    e = hipMalloc(&b.ptr, size);
  }
  CHECK(e == hipSuccess) << "hipMalloc(" << size << " bytes): " << hipGetErrorString(e);
  std::lock_guard<std::mutex> lk(mu_);
  dev_total_ += size;
  return b;
}

void MemoryPool::Return(const Block& b) {
  if (!b.ptr) return;
  std::lock_guard<std::mutex> lk(mu_);
  if (b.device < 0) {
    free_host_.insert(std::make_pair(b.size, b));
    host_unused_ += b.size;
  } else {
    free_dev_.insert(std::make_pair(std::make_pair(b.device, b.size), b));
    dev_unused_ += b.size;
  }
}

void MemoryPool::Clear() {
  std::lock_guard<std::mutex> lk(mu_);
  for (auto& kv : free_host_) {
    if (kv.second.pinned) (void)hipHostFree(kv.second.ptr);
    else std::free(kv.second.ptr);
    host_total_ -= kv.second.size;
  }
  for (auto& kv : free_dev_) {
    (void)hipFree(kv.second.ptr);
    dev_total_ -= kv.second.size;
  }
  free_host_.clear();
  free_dev_.clear();
  host_unused_ = 0;
  dev_unused_ = 0;
}

MemPoolState64 MemoryPool::GetState() {
  std::lock_guard<std::mutex> lk(mu_);
  MemPoolState64 s;
  s.gpu_mem = dev_total_;
  s.cpu_mem = host_total_;
  s.unused_gpu_mem = dev_unused_;
  s.unused_cpu_mem = host_unused_;
  return s;
}

// ---------------------------------------------------------------------------
// SyncedMemory
// ---------------------------------------------------------------------------

SyncedMemory::SyncedMemory(size_t size)
    : size_(size), head_(UNINITIALIZED), pool_(Context::Get().pool()), version_(0),
      h2d_epoch_(0), h2d_pending_(false) {}

SyncedMemory::~SyncedMemory() {
  // A pinned block that still feeds an asynchronous upload must not be recycled.
  if (h2d_pending_ && Context::Get().sync_epoch() == h2d_epoch_) {
    try {
      Context::Get().Sync();
    } catch (...) {
    }
  }
  pool_->Return(host_);
  pool_->Return(dev_);
}

void SyncedMemory::wait_pending_h2d() {
  if (h2d_pending_) {
    if (Context::Get().sync_epoch() == h2d_epoch_) Context::Get().Sync();
    h2d_pending_ = false;
  }
}

void SyncedMemory::to_cpu() {
  switch (head_) {
    case UNINITIALIZED:
      host_ = pool_->RequestHost(size_);
      head_ = HEAD_AT_CPU;
      break;
    case HEAD_AT_GPU: {
      if (!host_.ptr) host_ = pool_->RequestHost(size_);
      Context& ctx = Context::Get();
      HIP_CHECK(hipMemcpyAsync(host_.ptr, dev_.ptr, size_, hipMemcpyDeviceToHost, ctx.stream()));
      ctx.Sync();
      head_ = SYNCED;
      break;
    }
    case HEAD_AT_CPU:
    case SYNCED:
      break;
  }
}

void SyncedMemory::to_gpu() {
  CHECK(Context::gpu_available()) << "device memory requested but no HIP device is present";
  switch (head_) {
    case UNINITIALIZED:
      dev_ = pool_->RequestDevice(size_, Context::Get().device());
      head_ = HEAD_AT_GPU;
      break;
    case HEAD_AT_CPU: {
      if (!dev_.ptr) dev_ = pool_->RequestDevice(size_, Context::Get().device());
      Context& ctx = Context::Get();
      HIP_CHECK(hipMemcpyAsync(dev_.ptr, host_.ptr, size_, hipMemcpyHostToDevice, ctx.stream()));
      h2d_pending_ = true;
      h2d_epoch_ = ctx.sync_epoch();
      head_ = SYNCED;
      break;
    }
    case HEAD_AT_GPU:
    case SYNCED:
      break;
  }
}

const void* SyncedMemory::cpu_data() {
  to_cpu();
  return host_.ptr;
}

void* SyncedMemory::mutable_cpu_data() {
  to_cpu();
  wait_pending_h2d();  // the caller is about to overwrite the upload's source
  head_ = HEAD_AT_CPU;
  ++version_;
  return host_.ptr;
}

const void* SyncedMemory::gpu_data() {
  to_gpu();
  return dev_.ptr;
}

void* SyncedMemory::mutable_gpu_data() {
  to_gpu();
  head_ = HEAD_AT_GPU;
  ++version_;
  return dev_.ptr;
}

}  // namespace caffe

extern "C" void* mcCurrentStream(void) {
  try {
    return caffe::Context::Get().stream();
  } catch (const caffe::Error&) {
    return nullptr;
  }
}
