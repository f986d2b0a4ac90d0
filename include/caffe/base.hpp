/*
 * Common declarations of the Mini-Caffe host API, MI355X build.
 * Mirrors reference include/caffe/base.hpp:48-77 (real_t, DeviceMode, SetMode,
 * GPUAvailable, MemPoolState/MemPoolGetState/MemPoolClear).
 */
#ifndef CAFFE_BASE_HPP_
#define CAFFE_BASE_HPP_

#include <memory>
#include <string>
#include <vector>

#include "caffe/logging.hpp"

#define CAFFE_API __attribute__((visibility("default")))

#define DISABLE_COPY_AND_ASSIGN(classname)         \
 private:                                          \
  classname(const classname&) = delete;            \
  classname(classname&&) = delete;                 \
  classname& operator=(const classname&) = delete; \
  classname& operator=(classname&&) = delete

#define NOT_IMPLEMENTED LOG(FATAL) << "Not Implemented Yet"

namespace caffe {

using std::shared_ptr;
using std::string;
using std::vector;

typedef float real_t;

enum DeviceMode { CPU, GPU };

/*! \brief true when a HIP device is visible to this process */
CAFFE_API bool GPUAvailable();
/*!
 * \brief select mode and device for the calling thread
 * \param mode GPU runs the HIP path; CPU only builds and reshapes nets
 *        (this library carries no CPU arithmetic: Forward in CPU mode throws)
 * \param device HIP device id, ignored for CPU
 */
CAFFE_API void SetMode(DeviceMode mode, int device);

/*! \brief per-thread memory pool usage in bytes; the int fields saturate at INT_MAX */
struct MemPoolState {
  int gpu_mem;
  int cpu_mem;
  int unused_gpu_mem;
  int unused_cpu_mem;
};
CAFFE_API MemPoolState MemPoolGetState();
/*! \brief the same counters without the 2 GiB ceiling */
struct MemPoolState64 {
  long long gpu_mem;
  long long cpu_mem;
  long long unused_gpu_mem;
  long long unused_cpu_mem;
};
CAFFE_API MemPoolState64 MemPoolGetState64();
/*! \brief release every unused block of the calling thread's pool */
CAFFE_API void MemPoolClear();

}  // namespace caffe

#endif  // CAFFE_BASE_HPP_
