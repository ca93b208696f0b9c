// Entry point of the benchmark executable: harness flags first, then the benchmark runner
// (reference src/main.cpp:22-60: init(argc, argv) then Initialize / RunSpecifiedBenchmarks
// inside try/catch, with --benchmark_counters_tabular=true appended).
#include <cstdio>
#include <exception>
#include <string>
#include <vector>

#include "harness.hpp"
#include "minibench.hpp"

static int run_benchmark(int argc, char **argv) {
  try {
    benchmark::Initialize(&argc, argv);
    if (benchmark::ReportUnrecognizedArguments(argc, argv)) return 1;
    benchmark::RunSpecifiedBenchmarks();
  } catch (const std::exception &e) {
    std::fprintf(stderr, "ERROR:: Exception = %s\n", e.what());
    return 1;
  } catch (...) {
    std::fprintf(stderr, "ERROR:: Uncaught exception\n");
    return 1;
  }
  return 0;
}

int main(int argc, char **argv) {
  std::vector<char *> args(argv, argv + argc);
  static char tabular[] = "--benchmark_counters_tabular=true";
  args.push_back(tabular);
  int n = (int)args.size();
  harness::init_flags(&n, args.data());
  if (harness::flags().help) return 0;
  bool list_only = false;
  for (int i = 1; i < n; i++)
    if (std::string(args[i]).rfind("--benchmark_list_tests", 0) == 0) list_only = true;
  if (!list_only && !harness::init_device()) return 1;
  return run_benchmark(n, args.data());
}
