// extern "C" shim over Net / Blob / Profiler.  Every entry point catches
// caffe::Error (raised by CHECK / LOG(FATAL)) and reports it as -1 plus a
// per-thread message, like the reference's src/c_api.cpp:9-10,212-229; unlike
// the reference it also fences off std::exception so nothing unwinds into C.
#include "caffe/c_api.h"

#include <cstring>
#include <string>
#include <vector>

#include "caffe/caffe.hpp"
#include "device.hpp"
#include "proto.hpp"

namespace {

thread_local std::string g_last_error;
thread_local std::vector<int> g_shape_ret;
thread_local std::vector<const char*> g_names_ret;
thread_local std::vector<void*> g_handles_ret;

}  // namespace

#define API_BEGIN() try {
#define API_END()                         \
  }                                       \
  catch (const caffe::Error& e) {         \
    g_last_error = e.what();              \
    return -1;                            \
  }                                       \
  catch (const std::exception& e) {       \
    g_last_error = e.what();              \
    return -1;                            \
  }                                       \
  return 0;

extern "C" {

int CaffeBlobNum(BlobHandle blob) { return static_cast<caffe::Blob*>(blob)->num(); }
int CaffeBlobChannels(BlobHandle blob) { return static_cast<caffe::Blob*>(blob)->channels(); }
int CaffeBlobHeight(BlobHandle blob) { return static_cast<caffe::Blob*>(blob)->height(); }
int CaffeBlobWidth(BlobHandle blob) { return static_cast<caffe::Blob*>(blob)->width(); }
int CaffeBlobCount(BlobHandle blob) { return static_cast<caffe::Blob*>(blob)->count(); }

real_t* CaffeBlobData(BlobHandle blob) {
  try {
    return static_cast<caffe::Blob*>(blob)->mutable_cpu_data();
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return nullptr;
  }
}

int CaffeBlobReshape(BlobHandle blob, int shape_size, int* shape) {
  API_BEGIN();
  CHECK(blob != nullptr && shape_size >= 0 && (shape != nullptr || shape_size == 0))
      << "CaffeBlobReshape: bad argument";
  static_cast<caffe::Blob*>(blob)->Reshape(std::vector<int>(shape, shape + shape_size));
  API_END();
}

int CaffeBlobShape(BlobHandle blob, int* shape_size, int** shape) {
  API_BEGIN();
  g_shape_ret = static_cast<caffe::Blob*>(blob)->shape();
  *shape_size = static_cast<int>(g_shape_ret.size());
  *shape = g_shape_ret.data();
  API_END();
}

int CaffeNetCreate(const char* net_path, const char* model_path, NetHandle* net) {
  API_BEGIN();
  CHECK(net_path && model_path && net) << "CaffeNetCreate: null argument";
  std::unique_ptr<caffe::Net> n(new caffe::Net(std::string(net_path)));
  n->CopyTrainedLayersFrom(std::string(model_path));
  *net = n.release();
  API_END();
}

int CaffeNetCreateFromBuffer(const char* net_buffer, int nb_len, const char* model_buffer,
                             int mb_len, NetHandle* net) {
  API_BEGIN();
  CHECK(net_buffer && net && nb_len >= 0 && mb_len >= 0 && (model_buffer || mb_len == 0))
      << "CaffeNetCreateFromBuffer: bad argument";
  auto net_param = caffe::ReadTextNetParameterFromBuffer(net_buffer, nb_len);
  std::unique_ptr<caffe::Net> n(new caffe::Net(*net_param));
  if (mb_len > 0) {
    auto model_param = caffe::ReadBinaryNetParameterFromBuffer(model_buffer, mb_len);
    n->CopyTrainedLayersFrom(*model_param);
  }
  *net = n.release();
  API_END();
}

int CaffeNetDestroy(NetHandle net) {
  API_BEGIN();
  delete static_cast<caffe::Net*>(net);
  API_END();
}

int CaffeNetMarkOutput(NetHandle net, const char* name) {
  API_BEGIN();
  static_cast<caffe::Net*>(net)->MarkOutputs({std::string(name)});
  API_END();
}

int CaffeNetForward(NetHandle net) {
  API_BEGIN();
  static_cast<caffe::Net*>(net)->Forward();
  API_END();
}

int CaffeNetGetBlob(NetHandle net, const char* name, BlobHandle* blob) {
  API_BEGIN();
  *blob = static_cast<caffe::Net*>(net)->blob_by_name(name).get();
  API_END();
}

int CaffeNetListBlob(NetHandle net, int* n, const char*** names, BlobHandle** blobs) {
  API_BEGIN();
  caffe::Net* net_ = static_cast<caffe::Net*>(net);
  const auto& names_ = net_->blob_names();
  const auto& blobs_ = net_->blobs();
  g_names_ret.resize(names_.size());
  g_handles_ret.resize(blobs_.size());
  for (size_t i = 0; i < names_.size(); ++i) {
    g_names_ret[i] = names_[i].c_str();
    g_handles_ret[i] = blobs_[i].get();
  }
  *n = static_cast<int>(names_.size());
  *names = g_names_ret.data();
  *blobs = g_handles_ret.data();
  API_END();
}

int CaffeNetListParam(NetHandle net, int* n, const char*** names, BlobHandle** params) {
  API_BEGIN();
  caffe::Net* net_ = static_cast<caffe::Net*>(net);
  const auto& names_ = net_->param_names();
  const auto& params_ = net_->params();
  g_names_ret.resize(names_.size());
  g_handles_ret.resize(params_.size());
  for (size_t i = 0; i < names_.size(); ++i) {
    g_names_ret[i] = names_[i].c_str();
    g_handles_ret[i] = params_[i].get();
  }
  *n = static_cast<int>(names_.size());
  *names = g_names_ret.data();
  *params = g_handles_ret.data();
  API_END();
}

int CaffeProfilerEnable() {
  API_BEGIN();
  caffe::Profiler::Get()->TurnON();
  API_END();
}

int CaffeProfilerDisable() {
  API_BEGIN();
  caffe::Profiler::Get()->TurnOFF();
  API_END();
}

int CaffeProfilerScopeStart(const char* name) {
  API_BEGIN();
  caffe::Profiler::Get()->ScopeStart(name);
  API_END();
}

int CaffeProfilerScopeEnd() {
  API_BEGIN();
  caffe::Profiler::Get()->ScopeEnd();
  API_END();
}

int CaffeProfilerDump(const char* fn) {
  API_BEGIN();
  caffe::Profiler::Get()->DumpProfile(fn);
  API_END();
}

int CaffeGPUAvailable() { return caffe::GPUAvailable() ? 1 : 0; }

int CaffeSetMode(int mode, int device) {
  API_BEGIN();
  CHECK(mode == 0 || mode == 1) << "CaffeSetMode: mode must be 0 (CPU) or 1 (GPU)";
  caffe::SetMode(mode == 1 ? caffe::GPU : caffe::CPU, device);
  API_END();
}

const char* CaffeGetLastError() { return g_last_error.c_str(); }

int CaffeMemoryPoolClear() {
  API_BEGIN();
  caffe::MemPoolClear();
  API_END();
}

}  // extern "C"
