// Entry point of the benchmark executable.  Order of business, as in the reference's
// src/main.cpp:22-60: the harness takes its own flags off the command line, the device is
// selected, then the benchmark runner parses what is left and runs what the filter selects;
// counters are printed as table columns (--benchmark_counters_tabular=true is always on).
#include <cstdio>
#include <cstring>
#include <exception>
#include <vector>

#include "harness.hpp"
#include "minibench.hpp"

namespace {

// argv plus the switches this executable always passes to the runner
struct CommandLine {
  std::vector<char *> words;
  CommandLine(int argc, char **argv) : words(argv, argv + argc) {
    static char tabular_counters[] = "--benchmark_counters_tabular=true";
    words.push_back(tabular_counters);
  }
  bool has_prefix(const char *prefix) const {
    for (size_t i = 1; i < words.size(); i++)
      if (std::strncmp(words[i], prefix, std::strlen(prefix)) == 0) return true;
    return false;
  }
};

enum ExitCode { kDone = 0, kFailed = 1 };

ExitCode run_selected_benchmarks(CommandLine &cl) {
  int count = (int)cl.words.size();
  benchmark::Initialize(&count, cl.words.data());
  if (benchmark::ReportUnrecognizedArguments(count, cl.words.data())) return kFailed;
  benchmark::RunSpecifiedBenchmarks();
  return kDone;
}

}  // namespace

int main(int argc, char **argv) {
  CommandLine cl(argc, argv);
  int count = (int)cl.words.size();
  harness::init_flags(&count, cl.words.data());  // removes the harness's own flags
  cl.words.resize((size_t)count);
  if (harness::flags().help) return kDone;
  // listing the benchmark names needs no GPU
  if (!cl.has_prefix("--benchmark_list_tests") && !harness::init_device()) return kFailed;
  try {
    return run_selected_benchmarks(cl);
  } catch (const std::exception &failure) {
    std::fprintf(stderr, "ERROR:: Exception = %s\n", failure.what());
  } catch (...) {
    std::fprintf(stderr, "ERROR:: Uncaught exception\n");
  }
  return kFailed;
}
