// Runner behind minibench.hpp: iteration-count selection on manual time, Google-Benchmark
// style console table and JSON report.
#include "minibench.hpp"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <fstream>
#include <iostream>
#include <memory>
#include <regex>
#include <sstream>

#include <unistd.h>

namespace benchmark {

namespace {

double now_seconds() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

struct Flags {
  std::string filter = ".";
  bool list_tests = false;
  double min_time = 0.5;
  int repetitions = 1;
  std::string out, out_format = "json";
  bool counters_tabular = false;
};
Flags &flags() {
  static Flags f;
  return f;
}
std::vector<std::unique_ptr<internal::Benchmark>> &registry() {
  static std::vector<std::unique_ptr<internal::Benchmark>> r;
  return r;
}

bool parse_flag(const char *arg, const char *name, std::string *value) {
  const size_t n = std::strlen(name);
  if (std::strncmp(arg, "--", 2) != 0 || std::strncmp(arg + 2, name, n) != 0) return false;
  if (arg[2 + n] == '\0') {
    *value = "true";
    return true;
  }
  if (arg[2 + n] != '=') return false;
  *value = arg + 3 + n;
  return true;
}
bool truthy(const std::string &v) { return !(v == "false" || v == "0" || v == "no" || v == "off"); }

struct Run {
  std::string name;
  bool error = false;
  std::string error_message, label;
  uint64_t iterations = 0;
  double real_time = 0, cpu_time = 0;  // per iteration, in the benchmark's unit
  const char *unit = "ns";
  std::vector<std::pair<std::string, double>> counters;
};

const char *unit_name(TimeUnit u) { return u == kMillisecond ? "ms" : u == kMicrosecond ? "us" : "ns"; }
double unit_scale(TimeUnit u) { return u == kMillisecond ? 1e3 : u == kMicrosecond ? 1e6 : 1e9; }

std::string json_escape(const std::string &s) {
  std::string o;
  for (char c : s) {
    if (c == '"' || c == '\\') {
      o += '\\';
      o += c;
    } else if (c == '\n') {
      o += "\\n";
    } else {
      o += c;
    }
  }
  return o;
}

std::string human(double v) {
  char buf[64];
  const double a = std::fabs(v);
  if (a >= 1e12)
    std::snprintf(buf, sizeof buf, "%.4gT", v / 1e12);
  else if (a >= 1e9)
    std::snprintf(buf, sizeof buf, "%.4gG", v / 1e9);
  else if (a >= 1e6)
    std::snprintf(buf, sizeof buf, "%.4gM", v / 1e6);
  else if (a >= 1e3)
    std::snprintf(buf, sizeof buf, "%.4gk", v / 1e3);
  else
    std::snprintf(buf, sizeof buf, "%.4g", v);
  return buf;
}

}  // namespace

State::State(std::vector<int64_t> ranges, uint64_t max_iterations, bool manual_time) : ranges_(std::move(ranges)), max_iterations_(max_iterations), manual_(manual_time) {}

bool State::KeepRunning() {
  if (!started_) {
    started_ = true;
    if (skipped_) return false;
    running_ = true;
    t_start_ = now_seconds();
    if (max_iterations_ == 0) {
      running_ = false;
      return false;
    }
    return true;
  }
  if (skipped_) {
    running_ = false;
    return false;
  }
  ++done_;
  if (done_ < max_iterations_) return true;
  if (running_) real_seconds_ += now_seconds() - t_start_;
  running_ = false;
  return false;
}
void State::PauseTiming() {
  if (running_) {
    real_seconds_ += now_seconds() - t_start_;
    running_ = false;
  }
}
void State::ResumeTiming() {
  if (!running_ && started_ && !skipped_) {
    t_start_ = now_seconds();
    running_ = true;
  }
}
void State::SkipWithError(const char *msg) {
  if (!skipped_) error_ = msg ? msg : "";
  skipped_ = true;
}

namespace internal {
Benchmark *RegisterBenchmarkInternal(Benchmark *b) {
  registry().emplace_back(b);
  return b;
}
}  // namespace internal

void Initialize(int *argc, char **argv) {
  int out = 1;
  for (int i = 1; i < *argc; i++) {
    std::string v;
    Flags &f = flags();
    if (parse_flag(argv[i], "benchmark_filter", &v))
      f.filter = v;
    else if (parse_flag(argv[i], "benchmark_list_tests", &v))
      f.list_tests = truthy(v);
    else if (parse_flag(argv[i], "benchmark_min_time", &v))
      f.min_time = std::atof(v.c_str());
    else if (parse_flag(argv[i], "benchmark_repetitions", &v))
      f.repetitions = std::max(1, std::atoi(v.c_str()));
    else if (parse_flag(argv[i], "benchmark_out_format", &v))
      f.out_format = v;
    else if (parse_flag(argv[i], "benchmark_out", &v))
      f.out = v;
    else if (parse_flag(argv[i], "benchmark_counters_tabular", &v))
      f.counters_tabular = truthy(v);
    else if (parse_flag(argv[i], "benchmark_format", &v) || parse_flag(argv[i], "benchmark_color", &v) || parse_flag(argv[i], "benchmark_report_aggregates_only", &v) ||
             parse_flag(argv[i], "benchmark_display_aggregates_only", &v))
      ;  // accepted, no effect
    else
      argv[out++] = argv[i];
  }
  *argc = out;
}

bool ReportUnrecognizedArguments(int argc, char **argv) {
  for (int i = 1; i < argc; i++) std::fprintf(stderr, "%s: error: unrecognized command-line flag: %s\n", argv[0], argv[i]);
  return argc > 1;
}

static std::string instance_name(const internal::Benchmark &b, const std::vector<int64_t> &args) {
  std::string name = b.name_;
  for (size_t i = 0; i < args.size(); i++) {
    name += "/";
    if (i < b.arg_names_.size() && !b.arg_names_[i].empty()) name += b.arg_names_[i] + ":";
    name += std::to_string(args[i]);
  }
  if (b.manual_time_)
    name += "/manual_time";
  else if (b.real_time_)
    name += "/real_time";
  return name;
}

static Run run_instance(const internal::Benchmark &b, const std::vector<int64_t> &args, const std::string &name) {
  Run r;
  r.name = name;
  r.unit = unit_name(b.unit_);
  const double min_time = b.min_time_ > 0 ? b.min_time_ : flags().min_time;
  uint64_t iters = b.fixed_iterations_ ? b.fixed_iterations_ : 1;
  for (;;) {
    State st(args, iters, b.manual_time_);
    const double cpu0 = (double)std::clock() / CLOCKS_PER_SEC;
    b.fn_(st);
    const double cpu1 = (double)std::clock() / CLOCKS_PER_SEC;
    if (st.error_occurred()) {
      r.error = true;
      r.error_message = st.error_message();
      return r;
    }
    const double measured = b.manual_time_ ? st.manual_seconds() : st.real_seconds();
    const bool enough = b.fixed_iterations_ || measured >= min_time || iters >= 1000000000ull || st.real_seconds() >= 5.0 * std::max(min_time, 1e-9);
    if (enough || st.iterations() == 0) {
      const uint64_t n = std::max<uint64_t>(st.iterations(), 1);
      r.iterations = st.iterations();
      r.real_time = measured / n * unit_scale(b.unit_);
      r.cpu_time = (cpu1 - cpu0) / n * unit_scale(b.unit_);
      r.label = st.label();
      for (const auto &kv : st.counters) {
        double v = kv.second.value;
        // rates are per second of the measured (manual) time, as Google Benchmark computes them
        if (kv.second.flags & Counter::kIsRate) v = measured > 0 ? v / measured : 0.0;
        r.counters.emplace_back(kv.first, v);
      }
      if (st.items() > 0 && measured > 0) r.counters.emplace_back("items_per_second", st.items() / measured);
      if (st.bytes() > 0 && measured > 0) r.counters.emplace_back("bytes_per_second", st.bytes() / measured);
      return r;
    }
    // aim 40 % past the target, grow at most 10x per step (Google Benchmark's rule)
    double mult = measured > 0 ? min_time * 1.4 / measured : 10.0;
    mult = std::min(10.0, std::max(mult, 2.0));
    iters = std::max<uint64_t>(iters + 1, (uint64_t)std::llround(iters * mult));
  }
}

size_t RunSpecifiedBenchmarks() {
  const Flags &f = flags();
  std::regex re;
  try {
    re = std::regex(f.filter == "all" || f.filter.empty() ? "." : f.filter, std::regex::extended);
  } catch (const std::regex_error &e) {
    std::fprintf(stderr, "could not compile --benchmark_filter: %s\n", e.what());
    return 0;
  }
  struct Item {
    const internal::Benchmark *b;
    std::vector<int64_t> args;
    std::string name;
  };
  std::vector<Item> items;
  for (const auto &b : registry()) {
    std::vector<std::vector<int64_t>> argsets = b->args_;
    if (argsets.empty()) argsets.push_back({});
    for (const auto &a : argsets) {
      std::string name = instance_name(*b, a);
      if (std::regex_search(name, re)) items.push_back({b.get(), a, std::move(name)});
    }
  }
  if (f.list_tests) {
    for (const auto &it : items) std::printf("%s\n", it.name.c_str());
    return items.size();
  }
  size_t width = 10;
  for (const auto &it : items) width = std::max(width, it.name.size());
  char host[256] = "unknown";
  gethostname(host, sizeof host);
  std::time_t tt = std::time(nullptr);
  char date[64];
  std::strftime(date, sizeof date, "%Y-%m-%d %H:%M:%S", std::localtime(&tt));
  std::printf("%s\nRunning on %s\n", date, host);
  std::printf("%s\n", std::string(width + 60, '-').c_str());
  std::printf("%-*s %13s %13s %12s  %s\n", (int)width, "Benchmark", "Time", "CPU", "Iterations", "UserCounters...");
  std::printf("%s\n", std::string(width + 60, '-').c_str());

  std::vector<Run> runs;
  for (const auto &it : items) {
    for (int rep = 0; rep < f.repetitions; rep++) {
      Run r = run_instance(*it.b, it.args, it.name);
      if (r.error) {
        std::printf("%-*s ERROR OCCURRED: '%s'\n", (int)width, r.name.c_str(), r.error_message.c_str());
      } else {
        std::printf("%-*s %10.0f %s %10.0f %s %12llu ", (int)width, r.name.c_str(), r.real_time, r.unit, r.cpu_time, r.unit, (unsigned long long)r.iterations);
        for (const auto &c : r.counters) std::printf(" %s=%s", c.first.c_str(), human(c.second).c_str());
        if (!r.label.empty()) std::printf(" %s", r.label.c_str());
        std::printf("\n");
      }
      std::fflush(stdout);
      runs.push_back(std::move(r));
    }
  }
  if (!f.out.empty()) {
    std::ofstream o(f.out);
    o << "{\n  \"context\": {\n    \"date\": \"" << date << "\",\n    \"host_name\": \"" << json_escape(host) << "\",\n    \"executable\": \"bench\",\n    \"num_cpus\": "
      << sysconf(_SC_NPROCESSORS_ONLN) << ",\n    \"library_build_type\": \"release\"\n  },\n  \"benchmarks\": [\n";
    for (size_t i = 0; i < runs.size(); i++) {
      const Run &r = runs[i];
      o << "    {\n      \"name\": \"" << json_escape(r.name) << "\",\n";
      if (r.error) {
        o << "      \"error_occurred\": true,\n      \"error_message\": \"" << json_escape(r.error_message) << "\",\n";
      }
      o << "      \"iterations\": " << r.iterations << ",\n      \"real_time\": " << r.real_time << ",\n      \"cpu_time\": " << r.cpu_time << ",\n      \"time_unit\": \"" << r.unit << "\"";
      for (const auto &c : r.counters) {
        std::ostringstream v;
        v.precision(17);
        v << c.second;
        o << ",\n      \"" << json_escape(c.first) << "\": " << v.str();
      }
      o << "\n    }" << (i + 1 < runs.size() ? "," : "") << "\n";
    }
    o << "  ]\n}\n";
  }
  return runs.size();
}

}  // namespace benchmark
