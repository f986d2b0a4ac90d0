// Forward-pass timing of a network definition, with the command line and the
// output of the reference's own tool (reference tools/benchmark.cpp:7-39):
//
//   benchmark net.prototxt iterations gpu_id
//
// builds the net from the prototxt alone (parameters keep their constant
// fillers), runs `iterations` forward passes under the profiler, logs the wall
// time of each pass and writes the layer scopes to ./profile.json.  It is built
// against the public C++ headers only, as a check that sources written for the
// reference compile and link against this library unchanged.
#include <cstdlib>
#include <string>
#include <vector>

#include <caffe/net.hpp>
#include <caffe/profiler.hpp>

int main(int argc, char* argv[]) {
  CHECK_EQ(argc, 4) << "[Usage]: ./benchmark net.prototxt iterations gpu_id";
  const std::string proto = argv[1];
  const int iters = std::atoi(argv[2]);
  int gpu_id = std::atoi(argv[3]);
  LOG(INFO) << "net prototxt: " << proto;
  LOG(INFO) << "net forward iterations: " << iters;
  if (gpu_id >= 0 && caffe::GPUAvailable()) {
    caffe::SetMode(caffe::GPU, gpu_id);
    LOG(INFO) << "run on device " << gpu_id;
  } else {
    gpu_id = -1;
    LOG(INFO) << "no device selected: this library has no CPU arithmetic, Forward will refuse";
  }
  try {
    caffe::Net net(proto);
    caffe::Profiler* profiler = caffe::Profiler::Get();
    profiler->TurnON();
    std::vector<double> ms;
    for (int i = 0; i < iters; ++i) {
      const uint64_t tic = profiler->Now();
      net.Forward();
      const uint64_t toc = profiler->Now();
      ms.push_back((toc - tic) / 1000.);
      LOG(INFO) << "Forward costs " << ms.back() << " ms";
    }
    profiler->TurnOFF();
    profiler->DumpProfile("./profile.json");
    if (!ms.empty()) {
      double best = ms[0], sum = 0.;
      for (double v : ms) {
        best = v < best ? v : best;
        sum += v;
      }
      LOG(INFO) << "mean " << sum / ms.size() << " ms, best " << best << " ms over " << ms.size()
                << " passes (layer scopes synchronise the stream while the profiler is on)";
    }
  } catch (const std::exception& e) {
    LOG(INFO) << "failed: " << e.what();
    return 1;
  }
  return 0;
}
