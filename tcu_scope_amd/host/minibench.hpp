// A small benchmark runner that is source-compatible with the slice of Google Benchmark the
// tcu_scope harnesses use (Google Benchmark itself is not available offline):
//   static void NAME(benchmark::State &state) { for (auto _ : state) { ... state.SetIterationTime(s); } }
//   BENCHMARK(NAME) / BENCHMARK_TEMPLATE(NAME, targs...) ->Args({..})->ArgNames({..})->Apply(fn)->UseManualTime();
//   state.range(i), state.iterations(), state.PauseTiming(), state.ResumeTiming(),
//   state.SkipWithError(msg), state.counters (benchmark::Counter with kAvgThreadsRate ...)
//   benchmark::Initialize(&argc, argv); benchmark::RunSpecifiedBenchmarks();
// and with its command line: --benchmark_filter=<regex> --benchmark_list_tests
// --benchmark_min_time=<seconds> --benchmark_repetitions=<n> --benchmark_out=<file>
// --benchmark_out_format=json|console --benchmark_counters_tabular=true|false.
// Benchmark names follow Google Benchmark's grammar
//   FUNC<template argument text>/argname:value/.../manual_time
// because the plotting specs of the reference select series by regular expressions over
// those names (reference figures/spec/*.yml, tools/plot.py:101-128).
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <vector>

namespace benchmark {

class Counter {
 public:
  enum Flags { kDefaults = 0, kIsRate = 1, kAvgThreads = 2, kAvgThreadsRate = kIsRate | kAvgThreads };
  double value;
  Flags flags;
  Counter(double v = 0.0, Flags f = kDefaults) : value(v), flags(f) {}
  operator double() const { return value; }
};

enum TimeUnit { kNanosecond, kMicrosecond, kMillisecond };

class State {
 public:
  State(std::vector<int64_t> ranges, uint64_t max_iterations, bool manual_time);

  // range-for support: `for (auto _ : state)`
  struct __attribute__((unused)) Token {};
  struct Iterator {
    State *state;
    bool operator!=(const Iterator &) const { return state->KeepRunning(); }
    void operator++() {}
    Token operator*() const { return Token(); }
  };
  Iterator begin() { return Iterator{this}; }
  Iterator end() { return Iterator{this}; }

  bool KeepRunning();
  int64_t range(size_t i = 0) const { return ranges_.at(i); }
  uint64_t iterations() const { return done_; }
  void SetIterationTime(double seconds) { manual_seconds_ += seconds; }
  void PauseTiming();
  void ResumeTiming();
  void SkipWithError(const char *msg);
  void SetItemsProcessed(int64_t n) { items_ = n; }
  void SetBytesProcessed(int64_t n) { bytes_ = n; }
  void SetLabel(const std::string &l) { label_ = l; }
  bool error_occurred() const { return skipped_; }

  std::map<std::string, Counter> counters;

  // runner side
  double manual_seconds() const { return manual_seconds_; }
  double real_seconds() const { return real_seconds_; }
  const std::string &error_message() const { return error_; }
  const std::string &label() const { return label_; }
  int64_t items() const { return items_; }
  int64_t bytes() const { return bytes_; }

 private:
  std::vector<int64_t> ranges_;
  uint64_t max_iterations_, done_ = 0;
  bool manual_, started_ = false, skipped_ = false, running_ = false;
  double manual_seconds_ = 0.0, real_seconds_ = 0.0, t_start_ = 0.0;
  int64_t items_ = 0, bytes_ = 0;
  std::string error_, label_;
};

namespace internal {

class Benchmark {
 public:
  Benchmark(std::string name, std::function<void(State &)> fn) : name_(std::move(name)), fn_(std::move(fn)) {}
  Benchmark *Arg(int64_t x) { return Args({x}); }
  Benchmark *Args(const std::vector<int64_t> &args) {
    args_.push_back(args);
    return this;
  }
  Benchmark *ArgName(const std::string &n) { return ArgNames({n}); }
  Benchmark *ArgNames(const std::vector<std::string> &names) {
    arg_names_ = names;
    return this;
  }
  Benchmark *Apply(void (*fn)(Benchmark *)) {
    fn(this);
    return this;
  }
  Benchmark *UseManualTime() {
    manual_time_ = true;
    return this;
  }
  Benchmark *UseRealTime() {
    real_time_ = true;
    return this;
  }
  Benchmark *Unit(TimeUnit u) {
    unit_ = u;
    return this;
  }
  Benchmark *Iterations(uint64_t n) {
    fixed_iterations_ = n;
    return this;
  }
  Benchmark *MinTime(double s) {
    min_time_ = s;
    return this;
  }

  std::string name_;
  std::function<void(State &)> fn_;
  std::vector<std::vector<int64_t>> args_;
  std::vector<std::string> arg_names_;
  bool manual_time_ = false, real_time_ = false;
  TimeUnit unit_ = kNanosecond;
  uint64_t fixed_iterations_ = 0;
  double min_time_ = 0.0;
};

Benchmark *RegisterBenchmarkInternal(Benchmark *b);

}  // namespace internal

void Initialize(int *argc, char **argv);
bool ReportUnrecognizedArguments(int argc, char **argv);
size_t RunSpecifiedBenchmarks();

}  // namespace benchmark

#define BENCHMARK_PRIVATE_CONCAT2(a, b) a##b
#define BENCHMARK_PRIVATE_CONCAT(a, b) BENCHMARK_PRIVATE_CONCAT2(a, b)
#define BENCHMARK_PRIVATE_NAME(n) BENCHMARK_PRIVATE_CONCAT(_benchmark_, BENCHMARK_PRIVATE_CONCAT(__COUNTER__, n))
#define BENCHMARK_PRIVATE_DECLARE(n) static ::benchmark::internal::Benchmark *BENCHMARK_PRIVATE_NAME(n) __attribute__((unused))

#define BENCHMARK(n) BENCHMARK_PRIVATE_DECLARE(n) = (::benchmark::internal::RegisterBenchmarkInternal(new ::benchmark::internal::Benchmark(#n, n)))
#define BENCHMARK_TEMPLATE(n, ...) \
  BENCHMARK_PRIVATE_DECLARE(n) = (::benchmark::internal::RegisterBenchmarkInternal(new ::benchmark::internal::Benchmark(#n "<" #__VA_ARGS__ ">", n<__VA_ARGS__>)))
#define BENCHMARK_TEMPLATE1(n, a) BENCHMARK_TEMPLATE(n, a)
#define BENCHMARK_TEMPLATE2(n, a, b) BENCHMARK_TEMPLATE(n, a, b)
