/*
 * Nested-scope wall-clock profiler that dumps chrome://tracing JSON
 * (reference include/caffe/profiler.hpp:28-84, src/profiler.cpp:24-99).
 * Process singleton without locks: do not enable it while several threads run
 * nets.  While it is on, Net::Forward synchronises the HIP stream at every
 * layer boundary so that scopes measure device time, not launch time.
 */
#ifndef CAFFE_PROFILER_HPP_
#define CAFFE_PROFILER_HPP_

#include <cstdint>
#include <string>
#include <vector>

#include "caffe/base.hpp"

namespace caffe {

class CAFFE_API Profiler {
 public:
  static Profiler* Get();
  void TurnON();
  void TurnOFF();
  bool enabled() const { return state_ == kRunning; }
  void ScopeStart(const char* name);
  void ScopeEnd();
  /*! \brief write all closed scopes as chrome tracing "B"/"E" events */
  void DumpProfile(const char* fn) const;
  /*! \brief microseconds since the profiler was created */
  uint64_t Now() const;

 private:
  Profiler();
  enum State { kRunning, kNotRunning };
  struct Scope {
    std::string name;
    uint64_t start_microsec = 0;
    uint64_t end_microsec = 0;
  };
  State state_;
  uint64_t init_;
  std::vector<Scope> open_;
  std::vector<Scope> closed_;
  DISABLE_COPY_AND_ASSIGN(Profiler);
};

}  // namespace caffe

#endif  // CAFFE_PROFILER_HPP_
