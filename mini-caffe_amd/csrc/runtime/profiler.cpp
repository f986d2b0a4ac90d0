#include "caffe/profiler.hpp"

#include <chrono>
#include <fstream>

namespace caffe {

namespace {
uint64_t MicrosSinceEpoch() {
  return static_cast<uint64_t>(std::chrono::duration_cast<std::chrono::microseconds>(
                                   std::chrono::steady_clock::now().time_since_epoch())
                                   .count());
}
}  // namespace

Profiler::Profiler() : state_(kNotRunning), init_(MicrosSinceEpoch()) {}

Profiler* Profiler::Get() {
  static Profiler* inst = new Profiler();
  return inst;
}

void Profiler::TurnON() {
  CHECK(state_ == kNotRunning) << "Profiler is already running";
  state_ = kRunning;
}

void Profiler::TurnOFF() {
  CHECK(state_ == kRunning) << "Profiler is not running";
  CHECK(open_.empty()) << "Profiler has " << open_.size() << " unclosed scope(s)";
  state_ = kNotRunning;
}

uint64_t Profiler::Now() const { return MicrosSinceEpoch() - init_; }

// Nested scopes are named "outer:inner", as in the reference (src/profiler.cpp:37-45).
void Profiler::ScopeStart(const char* name) {
  if (state_ == kNotRunning) return;
  Scope s;
  s.name = open_.empty() ? std::string(name) : open_.back().name + ":" + name;
  s.start_microsec = Now();
  open_.push_back(s);
}

void Profiler::ScopeEnd() {
  if (state_ == kNotRunning) return;
  CHECK(!open_.empty()) << "ScopeEnd without a matching ScopeStart";
  Scope s = open_.back();
  open_.pop_back();
  s.end_microsec = Now();
  closed_.push_back(s);
}

void Profiler::DumpProfile(const char* fn) const {
  CHECK(open_.empty()) << "Profiler has " << open_.size() << " unclosed scope(s)";
  std::ofstream file(fn);
  CHECK(file.good()) << "cannot open " << fn << " for writing";
  file << "{\n  \"traceEvents\": [";
  bool first = true;
  for (const Scope& s : closed_) {
    for (int phase = 0; phase < 2; ++phase) {
      file << (first ? "\n" : ",\n");
      first = false;
      file << "    {\"name\": \"" << s.name << "\", \"cat\": \"category\", \"ph\": \""
           << (phase == 0 ? "B" : "E") << "\", \"ts\": "
           << (phase == 0 ? s.start_microsec : s.end_microsec) << ", \"pid\": 0, \"tid\": 0}";
    }
  }
  file << "\n  ],\n  \"displayTimeUnit\": \"ms\"\n}\n";
}

}  // namespace caffe
