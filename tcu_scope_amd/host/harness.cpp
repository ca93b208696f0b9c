#include "harness.hpp"

#include "../../include/tcu_scope_dev.h"  // --tcu_option

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <thread>

namespace harness {

// ---------------------------------------------------------------------------------------
// flags and device
// ---------------------------------------------------------------------------------------
Flags &flags() {
  static Flags f;
  return f;
}

static bool take(const char *arg, const char *name, std::string *value) {
  const size_t n = std::strlen(name);
  if (std::strncmp(arg, "--", 2) != 0 || std::strncmp(arg + 2, name, n) != 0) return false;
  if (arg[2 + n] == '\0') {
    *value = "1";
    return true;
  }
  if (arg[2 + n] != '=') return false;
  *value = arg + 3 + n;
  return true;
}

void init_flags(int *argc, char **argv) {
  int out = 1;
  Flags &f = flags();
  for (int i = 1; i < *argc; i++) {
    std::string v;
    if (take(argv[i], "cuda_device_id", &v))
      f.cuda_device_id = std::atoi(v.c_str());
    else if (take(argv[i], "tcu_input", &v))
      f.input = v;
    else if (take(argv[i], "tcu_verify", &v))
      f.verify = v;
    else if (take(argv[i], "tcu_seed", &v))
      f.seed = std::strtoull(v.c_str(), nullptr, 0);
    else if (take(argv[i], "tcu_out_buffers", &v))
      f.out_buffers = std::atoi(v.c_str());
    else if (take(argv[i], "tcu_option", &v))
      f.options.push_back(v);
    else if (take(argv[i], "v", &v))
      f.verbose = std::atoi(v.c_str());
    else if (take(argv[i], "help", &v) || std::strcmp(argv[i], "-h") == 0)
      f.help = true;
    else
      argv[out++] = argv[i];
  }
  *argc = out;
  if (f.help) {
    std::printf(
        "tcu_scope_amd bench\n"
        "  --benchmark_filter=<regex> --benchmark_list_tests --benchmark_min_time=<s> --benchmark_repetitions=<n>\n"
        "  --benchmark_out=<file> --benchmark_out_format=json --benchmark_counters_tabular=true\n"
        "  --cuda_device_id=<n>   device to run on (0 when absent)\n"
        "  --tcu_input=uniform|constant|grid   inputs: seeded uniform [-1,1) (default), the constant 0.001, or k/2048\n"
        "  --tcu_verify=auto|all|none          check results against a CPU fp64 sum before timing (auto: up to 2^26 elements)\n"
        "  --tcu_option=<name>:<value>         a tuning switch of the library (tcu_set_option), may be given several times\n"
        "  --tcu_out_buffers=<n>               output buffers the scan benchmarks' timed launches take in turn (default 3)\n"
        "  --tcu_seed=<n>  --v=<level>\n");
  }
}

bool init_device() {
  int rc = tcu_init(flags().cuda_device_id);
  if (rc != TCU_OK) {
    std::fprintf(stderr, "tcu_init failed: %s\n", tcu_last_error());
    return false;
  }
  for (const std::string &o : flags().options) {  // after tcu_init, which sets some of them from the device
    const size_t colon = o.find(':');
    if (colon == std::string::npos || tcu_set_option(o.substr(0, colon).c_str(), std::atoi(o.c_str() + colon + 1)) != TCU_OK) {
      std::fprintf(stderr, "--tcu_option=%s: %s\n", o.c_str(), colon == std::string::npos ? "expected <name>:<value>" : tcu_last_error());
      return false;
    }
  }
  int cus = 0, wave = 0, lds = 0, gfx950 = 0;
  tcu_device_info(&cus, &wave, &lds, &gfx950);
  if (flags().verbose) std::printf("device: %d compute units, wavefront %d, %d bytes LDS, gfx950=%d; host threads: %u\n", cus, wave, lds, gfx950, std::thread::hardware_concurrency());
  return true;
}

void check_hip(hipError_t e, const char *expr, const char *file, int line) {
  if (e == hipSuccess) return;
  std::string msg = std::string(hipGetErrorString(e)) + " in " + expr + " at " + file + ":" + std::to_string(line);
  std::fprintf(stderr, "HIP error: %s\n", msg.c_str());
  throw hip_error(msg);
}
void check_tcu(int status, const char *expr) {
  if (status == TCU_OK) return;
  std::string msg = std::string(tcu_last_error());
  if (status == TCU_ERR_UNSUPPORTED) throw unsupported(msg);
  throw std::runtime_error(msg + " (" + expr + ")");
}

DeviceBuffer::DeviceBuffer(size_t bytes) : n_(bytes) { PRINT_IF_ERROR(hipMalloc(&p_, bytes ? bytes : 16)); }
DeviceBuffer::~DeviceBuffer() {
  if (p_) (void)hipFree(p_);
}
EventPair::EventPair() {
  PRINT_IF_ERROR(hipEventCreate(&a_));
  PRINT_IF_ERROR(hipEventCreate(&b_));
}
EventPair::~EventPair() {
  (void)hipEventDestroy(a_);
  (void)hipEventDestroy(b_);
}
void EventPair::start() { PRINT_IF_ERROR(hipEventRecord(a_, nullptr)); }
float EventPair::stop_ms() {
  PRINT_IF_ERROR(hipEventRecord(b_, nullptr));
  PRINT_IF_ERROR(hipEventSynchronize(b_));
  float ms = 0.0f;
  PRINT_IF_ERROR(hipEventElapsedTime(&ms, a_, b_));
  return ms;
}

// ---------------------------------------------------------------------------------------
// fp16 on the host
// ---------------------------------------------------------------------------------------
float half_to_float(uint16_t h) {
  union {
    uint32_t u;
    float f;
  } o, magic;
  magic.u = 113u << 23;
  const uint32_t shifted_exp = 0x7c00u << 13;
  o.u = ((uint32_t)h & 0x7fffu) << 13;
  const uint32_t e = o.u & shifted_exp;
  o.u += (127u - 15u) << 23;
  if (e == shifted_exp) {
    o.u += (128u - 16u) << 23;
  } else if (e == 0) {
    o.u += 1u << 23;
    o.f -= magic.f;
  }
  o.u |= ((uint32_t)h & 0x8000u) << 16;
  return o.f;
}
uint16_t float_to_half(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u, a = x & 0x7fffffffu;
  if (a >= 0x7f800000u) return (uint16_t)(sign | (a > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  if (a < 0x33000001u) return (uint16_t)sign;
  const int e = (int)(a >> 23) - 127;
  uint32_t man = (a & 0x7fffffu) | 0x800000u, base = 0;
  int shift = 13;
  if (e < -14) {
    shift = -e - 1;
  } else {
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q++;
  return (uint16_t)(sign | (base + q));
}
static double ulp_half(double v) {
  const double a = std::fabs(v);
  if (!(a >= 6.103515625e-05)) return std::ldexp(1.0, -24);
  if (a >= 32768.0) return 32.0;
  int e;
  (void)std::frexp(a, &e);
  return std::ldexp(1.0, e - 11);
}

// ---------------------------------------------------------------------------------------
// inputs and verification
// ---------------------------------------------------------------------------------------
void fill_input(void *d, size_t n, uint64_t seed) {
  const std::string &in = flags().input;
  if (in == "constant") {
    TCU_CHECK(tcu_fill_f16(d, 0.001f, n, nullptr));  // the reference's cuda_memory_set(d_in, 0.001f, n)
  } else if (in == "grid") {
    TCU_CHECK(tcu_generate_f16(d, n, seed, TCU_DIST_GRID, 0, nullptr));
  } else if (in == "uniform") {
    TCU_CHECK(tcu_generate_f16(d, n, seed, TCU_DIST_UNIFORM, 0, nullptr));
  } else {
    throw std::runtime_error("--tcu_input must be uniform, constant or grid");
  }
}
bool should_verify(size_t num_elements) {
  const std::string &v = flags().verify;
  if (v == "none" || v == "0") return false;
  if (v == "all" || v == "1") return true;
  return num_elements <= ((size_t)1 << 26);
}

static void check_value(uint16_t got, double ref, size_t segment_size, size_t index, const char *what, size_t *errors, std::string *first) {
  const double allow = 2.0 * ulp_half(ref) + 1e-3 * std::sqrt((double)segment_size);
  bool ok;
  if ((got & 0x7fffu) == 0x7c00u) {
    const double lim = 65520.0 - (64.0 + 1e-3 * std::sqrt((double)segment_size));
    ok = (got & 0x8000u) ? ref <= -lim : ref >= lim;
  } else if ((got & 0x7fffu) > 0x7c00u) {
    ok = false;
  } else {
    ok = std::fabs((double)half_to_float(got) - ref) <= allow;
  }
  if (!ok) {
    if (*errors == 0) {
      char buf[256];
      std::snprintf(buf, sizeof buf, "%s: expected %.9g, got out[%zu] = %.9g (allowed %.3g)", what, ref, index, (double)half_to_float(got), allow);
      *first = buf;
    }
    ++*errors;
  }
}

void verify_seg_reduce(const void *d_in, const void *d_out, size_t num_segments, size_t segment_size, const char *what) {
  const size_t n = num_segments * segment_size;
  std::vector<uint16_t> in(n), out(num_segments);
  PRINT_IF_ERROR(hipMemcpy(in.data(), d_in, n * 2, hipMemcpyDeviceToHost));
  PRINT_IF_ERROR(hipMemcpy(out.data(), d_out, num_segments * 2, hipMemcpyDeviceToHost));
  size_t errors = 0;
  std::string first;
  for (size_t j = 0; j < num_segments; j++) {
    double correct_segment_sum = 0;
    for (size_t i = 0; i < segment_size; i++) correct_segment_sum += half_to_float(in[j * segment_size + i]);
    check_value(out[j], correct_segment_sum, segment_size, j, what, &errors, &first);
  }
  if (errors) throw std::runtime_error(first + "; " + std::to_string(errors) + " errors");
}
void verify_seg_scan(const void *d_in, const void *d_out, size_t num_segments, size_t segment_size, const char *what) {
  const size_t n = num_segments * segment_size;
  std::vector<uint16_t> in(n), out(n);
  PRINT_IF_ERROR(hipMemcpy(in.data(), d_in, n * 2, hipMemcpyDeviceToHost));
  PRINT_IF_ERROR(hipMemcpy(out.data(), d_out, n * 2, hipMemcpyDeviceToHost));
  size_t errors = 0;
  std::string first;
  for (size_t j = 0; j < num_segments; j++) {
    double running = 0;
    for (size_t i = 0; i < segment_size; i++) {
      running += half_to_float(in[j * segment_size + i]);
      check_value(out[j * segment_size + i], running, segment_size, j * segment_size + i, what, &errors, &first);
    }
  }
  if (errors) throw std::runtime_error(first + "; " + std::to_string(errors) + " errors");
}

// ---------------------------------------------------------------------------------------
// timed loops
// ---------------------------------------------------------------------------------------
template <class Body>
static void guarded(benchmark::State &state, Body body) {
  try {
    body();
  } catch (const unsupported &e) {
    state.SkipWithError(e.what());
  } catch (const std::exception &e) {
    state.SkipWithError(e.what());
  } catch (...) {
    state.SkipWithError("unknown exception");
  }
}

// Output buffers of the scan benchmarks that the timed launches take in turn (--tcu_out_buffers, default 3): a
// launch then never rewrites lines that the launch before it left dirty in the 256 MiB memory-side cache, so every
// byte a kernel writes has to reach HBM at the rate it is written.  The reference writes one d_out
// (src/prefixsum/seg_wmma_256n.cu:12-222); its V100 has no such cache.
class RotatingOutputs {
 public:
  explicit RotatingOutputs(size_t bytes) {
    int n = flags().out_buffers < 1 ? 1 : flags().out_buffers;
    while (n > 1 && (double)bytes * n > 24.0 * 1024 * 1024 * 1024) n--;
    for (int i = 0; i < n; i++) bufs_.emplace_back(new DeviceBuffer(bytes));
  }
  void *first() const { return bufs_[0]->get(); }
  void *next() { return bufs_[turn_++ % bufs_.size()]->get(); }
  size_t count() const { return bufs_.size(); }

 private:
  std::vector<std::unique_ptr<DeviceBuffer>> bufs_;
  size_t turn_ = 0;
};

static void set_common_counters(benchmark::State &state, size_t num_segments, size_t segment_size, size_t num_elements, int waves_per_block, double bytes_per_iteration) {
  state.counters.insert({{"num_segments", (double)num_segments},
                         {"segment_size", (double)segment_size},
                         {"num_elements", (double)num_elements},
                         {"warps_per_block", (double)waves_per_block},
                         {"flops", {state.iterations() * 1.0 * num_elements, benchmark::Counter::kAvgThreadsRate}},
                         {"bytes_per_second", {state.iterations() * bytes_per_iteration, benchmark::Counter::kAvgThreadsRate}},
                         {"hbm_peak_fraction", {state.iterations() * bytes_per_iteration / 8e12, benchmark::Counter::kAvgThreadsRate}}});
}

// segmented benchmarks take (num_segments, segment_size[, ...]); the TUNE argument sets put
// base_segment_size and max_elements_log2 after them
void run_seg_reduce(benchmark::State &state, int variant, int tiles_per_wave, int waves_per_block, const char *name) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1);
    const size_t num_elements = num_segments * segment_size;
    const int nin = num_elements <= ((size_t)1 << 29) ? 2 : 1;  // two inputs alternate so that none is served from the Infinity Cache
    DeviceBuffer in[2] = {DeviceBuffer(num_elements * 2), DeviceBuffer(nin == 2 ? num_elements * 2 : 16)};
    DeviceBuffer out(num_segments * 2);
    for (int i = 0; i < nin; i++) fill_input(in[i].get(), num_elements, flags().seed + i);
    TCU_CHECK(tcu_seg_reduce_f16(in[0].get(), out.get(), num_segments, segment_size, variant, tiles_per_wave, waves_per_block, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) verify_seg_reduce(in[0].get(), out.get(), num_segments, segment_size, name);
    EventPair ev;
    size_t it = 0;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_seg_reduce_f16(in[it++ % nin].get(), out.get(), num_segments, segment_size, variant, tiles_per_wave, waves_per_block, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, num_segments, segment_size, num_elements, waves_per_block, 2.0 * num_elements + 2.0 * num_segments);
  });
}

void run_seg_reduce_offsets(benchmark::State &state, bool pass_expected_size, const char *name) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1);
    const size_t num_elements = num_segments * segment_size;
    if (num_elements >= ((size_t)1 << 31)) {
      state.SkipWithError("offsets are 32-bit integers");
      return;
    }
    const int nin = num_elements <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(num_elements * 2), DeviceBuffer(nin == 2 ? num_elements * 2 : 16)};
    DeviceBuffer out(num_segments * 2), offsets((num_segments + 1) * sizeof(int));
    for (int i = 0; i < nin; i++) fill_input(in[i].get(), num_elements, flags().seed + i);
    {
      std::vector<int> h(num_segments + 1);
      for (size_t j = 0; j <= num_segments; j++) h[j] = (int)(j * segment_size);
      PRINT_IF_ERROR(hipMemcpy(offsets.get(), h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    }
    const int *off = static_cast<const int *>(offsets.get());
    const size_t expected = pass_expected_size ? segment_size : 0;
    TCU_CHECK(tcu_seg_reduce_offsets_f16(in[0].get(), out.get(), num_segments, off, off + 1, 32, expected, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) verify_seg_reduce(in[0].get(), out.get(), num_segments, segment_size, name);
    EventPair ev;
    size_t it = 0;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_seg_reduce_offsets_f16(in[it++ % nin].get(), out.get(), num_segments, off, off + 1, 32, expected, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, num_segments, segment_size, num_elements, 0, 2.0 * num_elements + 2.0 * num_segments + 4.0 * num_segments);
  });
}

void run_seg_scan_offsets(benchmark::State &state, const char *name) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1);
    const size_t num_elements = num_segments * segment_size;
    if (num_elements >= ((size_t)1 << 31)) {
      state.SkipWithError("offsets are 32-bit integers");
      return;
    }
    const int nin = num_elements <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(num_elements * 2), DeviceBuffer(nin == 2 ? num_elements * 2 : 16)};
    DeviceBuffer offsets((num_segments + 1) * sizeof(int));
    RotatingOutputs out(num_elements * 2);
    for (int i = 0; i < nin; i++) fill_input(in[i].get(), num_elements, flags().seed + i);
    {
      std::vector<int> h(num_segments + 1);
      for (size_t j = 0; j <= num_segments; j++) h[j] = (int)(j * segment_size);
      PRINT_IF_ERROR(hipMemcpy(offsets.get(), h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    }
    const int *off = static_cast<const int *>(offsets.get());
    TCU_CHECK(tcu_seg_scan_offsets_f16(in[0].get(), out.first(), num_segments, off, off + 1, 32, segment_size, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) verify_seg_scan(in[0].get(), out.first(), num_segments, segment_size, name);
    EventPair ev;
    size_t it = 0;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_seg_scan_offsets_f16(in[it++ % nin].get(), out.next(), num_segments, off, off + 1, 32, segment_size, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, num_segments, segment_size, num_elements, 0, 4.0 * num_elements + 4.0 * num_segments);
    state.counters.insert({"output_buffers", (double)out.count()});
  });
}

void run_seg_scan(benchmark::State &state, int variant, int tiles_per_wave, int waves_per_block, bool with_totals, const char *name) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1);
    const size_t num_elements = num_segments * segment_size;
    const int nin = num_elements <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(num_elements * 2), DeviceBuffer(nin == 2 ? num_elements * 2 : 16)};
    DeviceBuffer totals(with_totals ? num_segments * 2 : 16);
    RotatingOutputs out(num_elements * 2);
    for (int i = 0; i < nin; i++) fill_input(in[i].get(), num_elements, flags().seed + i);
    void *tp = with_totals ? totals.get() : nullptr;
    TCU_CHECK(tcu_seg_scan_f16(in[0].get(), out.first(), tp, num_segments, segment_size, variant, tiles_per_wave, waves_per_block, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) {
      verify_seg_scan(in[0].get(), out.first(), num_segments, segment_size, name);
      if (with_totals) verify_seg_reduce(in[0].get(), totals.get(), num_segments, segment_size, name);
    }
    EventPair ev;
    size_t it = 0;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_seg_scan_f16(in[it++ % nin].get(), out.next(), tp, num_segments, segment_size, variant, tiles_per_wave, waves_per_block, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, num_segments, segment_size, num_elements, waves_per_block, 4.0 * num_elements);
    state.counters.insert({"output_buffers", (double)out.count()});
  });
}

void run_full_reduce(benchmark::State &state, int strategy, size_t segment_size, int waves_per_block, const char *name) {
  guarded(state, [&] {
    const size_t num_elements = state.range(0);
    if (strategy == TCU_FULL_MULTI_KERNEL && segment_size && num_elements % segment_size) {
      state.SkipWithError("num_elements must be multiples of SEGMENT_SIZE");
      return;
    }
    size_t ws_bytes = 0;
    TCU_CHECK(tcu_full_reduce_f16(nullptr, nullptr, num_elements, nullptr, &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
    DeviceBuffer in(num_elements * 2), out(16), ws(ws_bytes);
    fill_input(in.get(), num_elements, flags().seed);
    TCU_CHECK(tcu_full_reduce_f16(in.get(), out.get(), num_elements, ws.get(), &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) verify_seg_reduce(in.get(), out.get(), 1, num_elements, name);
    EventPair ev;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_full_reduce_f16(in.get(), out.get(), num_elements, ws.get(), &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, segment_size ? num_elements / segment_size : 1, segment_size, num_elements, waves_per_block, 2.0 * num_elements);
  });
}

void run_full_scan(benchmark::State &state, int strategy, size_t segment_size, int waves_per_block, const char *name) {
  guarded(state, [&] {
    const size_t num_elements = state.range(0);
    if (strategy == TCU_FULL_MULTI_KERNEL && segment_size && num_elements % segment_size) {
      state.SkipWithError("num_elements must be multiples of SEGMENT_SIZE");
      return;
    }
    size_t ws_bytes = 0;
    TCU_CHECK(tcu_full_scan_f16(nullptr, nullptr, num_elements, nullptr, &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
    DeviceBuffer in(num_elements * 2), ws(ws_bytes);
    RotatingOutputs out(num_elements * 2);
    fill_input(in.get(), num_elements, flags().seed);
    TCU_CHECK(tcu_full_scan_f16(in.get(), out.first(), num_elements, ws.get(), &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(num_elements)) verify_seg_scan(in.get(), out.first(), 1, num_elements, name);
    EventPair ev;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_full_scan_f16(in.get(), out.next(), num_elements, ws.get(), &ws_bytes, strategy, segment_size, waves_per_block, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    set_common_counters(state, segment_size ? num_elements / segment_size : 1, segment_size, num_elements, waves_per_block, 4.0 * num_elements);
    state.counters.insert({"output_buffers", (double)out.count()});
  });
}

void run_gemv(benchmark::State &state, int variant, const char *name, bool half_out, bool col_major) {
  guarded(state, [&] {
    const size_t M = state.range(0), K = state.range(1);
    const float alpha = 1.0f, beta = 0.0f;
    const size_t out_size = half_out ? 2 : 4;  // bytes per element of y
    const auto gemv = [half_out, col_major](const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
      if (col_major) return half_out ? tcu_gemv_col_major_f16_f16(A, M, x, y, M, K, alpha, beta, stream) : tcu_gemv_col_major_f16_f32(A, M, x, y, M, K, alpha, beta, stream);
      return half_out ? tcu_gemv_f16_f16(A, x, y, M, K, alpha, beta, variant, stream) : tcu_gemv_f16_f32(A, x, y, M, K, alpha, beta, variant, stream);
    };
    DeviceBuffer A(M * K * 2), x(K * 2), y(M * out_size);
    TCU_CHECK(tcu_generate_f16(A.get(), M * K, flags().seed, TCU_DIST_NORMAL, 0, nullptr));
    TCU_CHECK(tcu_generate_f16(x.get(), K, flags().seed + 1, TCU_DIST_NORMAL, 0, nullptr));
    PRINT_IF_ERROR(hipMemset(y.get(), 0, M * out_size));
    TCU_CHECK(gemv(A.get(), x.get(), y.get(), M, K, alpha, beta, variant, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(M * K)) {
      std::vector<uint16_t> hA(M * K), hx(K);
      std::vector<float> hy(M);
      PRINT_IF_ERROR(hipMemcpy(hA.data(), A.get(), M * K * 2, hipMemcpyDeviceToHost));
      PRINT_IF_ERROR(hipMemcpy(hx.data(), x.get(), K * 2, hipMemcpyDeviceToHost));
      if (half_out) {
        std::vector<uint16_t> raw(M);
        PRINT_IF_ERROR(hipMemcpy(raw.data(), y.get(), M * 2, hipMemcpyDeviceToHost));
        for (size_t m = 0; m < M; m++) hy[m] = half_to_float(raw[m]);
      } else {
        PRINT_IF_ERROR(hipMemcpy(hy.data(), y.get(), M * 4, hipMemcpyDeviceToHost));
      }
      for (size_t m = 0; m < M; m++) {
        double s = 0;
        for (size_t k = 0; k < K; k++) s += (double)half_to_float(hA[col_major ? k * M + m : m * K + k]) * half_to_float(hx[k]);
        if (std::fabs(hy[m] - s) > 1e-2 * std::max(std::fabs(s), std::sqrt((double)K))) throw std::runtime_error(std::string(name) + ": row " + std::to_string(m) + " differs from the fp64 dot product");
      }
    }
    EventPair ev;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(gemv(A.get(), x.get(), y.get(), M, K, alpha, beta, variant, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    const double bytes = 2.0 * M * K + 2.0 * K + (double)out_size * M;
    state.counters.insert({{"M", (double)M},
                           {"N", (double)K},
                           {"flops", {state.iterations() * 2.0 * M * K, benchmark::Counter::kAvgThreadsRate}},
                           {"bytes_per_second", {state.iterations() * bytes, benchmark::Counter::kAvgThreadsRate}},
                           {"hbm_peak_fraction", {state.iterations() * bytes / 8e12, benchmark::Counter::kAvgThreadsRate}}});
  });
}

void run_gemm(benchmark::State &state, int variant, const char *name, bool half_out) {
  guarded(state, [&] {
    const size_t M = state.range(0), N = state.range(1), K = state.range(2);
    // the reference's values (src/gemm/wmma.cu:575-576), rounded to fp16 for the fp16-output
    // benchmark as there (src/gemm/wmma.cu:679-680)
    const float alpha = half_out ? half_to_float(float_to_half(1.1f)) : 1.1f, beta = half_out ? half_to_float(float_to_half(1.2f)) : 1.2f;
    const size_t out_size = half_out ? 2 : 4;  // bytes per element of C and D
    const auto gemm = half_out ? tcu_gemm_f16_f16 : tcu_gemm_f16_f32;
    // The reference's argument list starts at 16^3, below the tiles of its own kernels (128 x 128 for compute_gemm,
    // 16 x 16 x 16 fragments on a fixed grid for the naive one), which then compute nothing or part of the product.
    // Here such sizes take whatever kernel fits (AUTO), so that every registered instance yields a checked product.
    if ((variant == TCU_VARIANT_BLOCK_LDS && (M % 128 || N % 128 || K % 32)) || (variant == TCU_VARIANT_MFMA_16N && (M % 32 || N % 32 || K % 16))) variant = TCU_VARIANT_AUTO;
    DeviceBuffer A(M * K * 2), B(N * K * 2), C(M * N * out_size), D(M * N * out_size);
    TCU_CHECK(tcu_generate_f16(A.get(), M * K, flags().seed, TCU_DIST_NORMAL, 0, nullptr));
    TCU_CHECK(tcu_generate_f16(B.get(), N * K, flags().seed + 1, TCU_DIST_NORMAL, 0, nullptr));
    PRINT_IF_ERROR(hipMemset(C.get(), 0, M * N * out_size));
    TCU_CHECK(gemm(A.get(), B.get(), C.get(), D.get(), M, N, K, alpha, beta, variant, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (should_verify(M * K) && M * N * K <= ((size_t)1 << 31)) {
      std::vector<uint16_t> hA(M * K), hB(N * K);
      std::vector<float> hD(M * N);
      PRINT_IF_ERROR(hipMemcpy(hA.data(), A.get(), M * K * 2, hipMemcpyDeviceToHost));
      PRINT_IF_ERROR(hipMemcpy(hB.data(), B.get(), N * K * 2, hipMemcpyDeviceToHost));
      if (half_out) {
        std::vector<uint16_t> raw(M * N);
        PRINT_IF_ERROR(hipMemcpy(raw.data(), D.get(), M * N * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < M * N; i++) hD[i] = half_to_float(raw[i]);
      } else {
        PRINT_IF_ERROR(hipMemcpy(hD.data(), D.get(), M * N * 4, hipMemcpyDeviceToHost));
      }
      for (size_t m = 0; m < M; m++)
        for (size_t n = 0; n < N; n++) {
          double s = 0;
          for (size_t k = 0; k < K; k++) s += (double)half_to_float(hA[m * K + k]) * half_to_float(hB[n * K + k]);
          s *= alpha;
          if (std::fabs(hD[m * N + n] - s) > 1e-2 * std::max(std::fabs(s), std::sqrt((double)K))) throw std::runtime_error(std::string(name) + ": element differs from the fp64 product");
        }
    }
    EventPair ev;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(gemm(A.get(), B.get(), C.get(), D.get(), M, N, K, alpha, beta, variant, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    state.counters.insert({{"M", (double)M},
                           {"N", (double)N},
                           {"K", (double)K},
                           {"flops", {state.iterations() * 2.0 * M * N * K, benchmark::Counter::kAvgThreadsRate}},
                           {"mfma_peak_fraction", {state.iterations() * 2.0 * M * N * K / 2.5e15, benchmark::Counter::kAvgThreadsRate}}});
  });
}

// ---------------------------------------------------------------------------------------
// accuracy comparisons (reference src/gemm/accuracy.cu:178-275, src/gemv/accuracy.cu:215-330):
// fp32 values uniform in [0, 1) are narrowed to fp16 on the device, two computations of the
// same product are compared element by element under the reference's rule (ratio within
// 1.0001 and difference within 1e-5), and the number of violations is reported as a counter.
// ---------------------------------------------------------------------------------------
static void fill_uniform01_f32(std::vector<float> &v, uint64_t seed) {
  for (size_t i = 0; i < v.size(); i++) {
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    v[i] = (float)(z >> 40) * (1.0f / 16777216.0f);
  }
}
struct Agreement {
  size_t errors = 0;
  double max_abs = 0, max_rel = 0;
  void add(float v1, float v2) {
    const double d = std::fabs((double)v1 - (double)v2);
    if (v1 / v2 > 1.0001 || v2 / v1 > 1.0001 || d > 1e-5) errors++;
    max_abs = std::max(max_abs, d);
    const double m = std::max(std::fabs((double)v1), std::fabs((double)v2));
    if (m > 0) max_rel = std::max(max_rel, d / m);
  }
};
// narrows `host` to fp16 on the device (the reference's convertFp32ToFp16 step)
static void upload_as_f16(const std::vector<float> &host, DeviceBuffer &f16) {
  DeviceBuffer f32(host.size() * 4);
  PRINT_IF_ERROR(hipMemcpy(f32.get(), host.data(), host.size() * 4, hipMemcpyHostToDevice));
  TCU_CHECK(tcu_convert_f32_to_f16(f16.get(), f32.get(), host.size(), nullptr));
  PRINT_IF_ERROR(hipDeviceSynchronize());
}

void run_gemm_accuracy(benchmark::State &state, const char *name) {
  guarded(state, [&] {
    const size_t M = state.range(0), N = state.range(1), K = state.range(2);
    if (M * N > ((size_t)1 << 26)) throw unsupported(std::string(name) + ": outputs beyond 2^26 elements are not compared on the host");
    const float alpha = 1.1f, beta = 1.2f;
    std::vector<float> hA(M * K), hB(N * K), hC(M * N);
    fill_uniform01_f32(hA, flags().seed);
    fill_uniform01_f32(hB, flags().seed + 1);
    fill_uniform01_f32(hC, flags().seed + 2);
    DeviceBuffer A(M * K * 2), B(N * K * 2), C(M * N * 4), D_direct(M * N * 4), D_tiled(M * N * 4);
    upload_as_f16(hA, A);
    upload_as_f16(hB, B);
    PRINT_IF_ERROR(hipMemcpy(C.get(), hC.data(), M * N * 4, hipMemcpyHostToDevice));
    // first: one tile per wave straight from global memory; second: the LDS-tiled kernel
    TCU_CHECK(tcu_gemm_f16_f32(A.get(), B.get(), C.get(), D_direct.get(), M, N, K, alpha, beta, TCU_VARIANT_MFMA_16N, nullptr));
    EventPair ev;
    for (auto _ : state) {
      ev.start();
      TCU_CHECK(tcu_gemm_f16_f32(A.get(), B.get(), C.get(), D_tiled.get(), M, N, K, alpha, beta, TCU_VARIANT_AUTO, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    std::vector<float> h1(M * N), h2(M * N);
    PRINT_IF_ERROR(hipMemcpy(h1.data(), D_direct.get(), M * N * 4, hipMemcpyDeviceToHost));
    PRINT_IF_ERROR(hipMemcpy(h2.data(), D_tiled.get(), M * N * 4, hipMemcpyDeviceToHost));
    Agreement ag;
    for (size_t i = 0; i < M * N; i++) ag.add(h1[i], h2[i]);
    state.counters.insert({{"M", (double)M}, {"N", (double)N}, {"K", (double)K}, {"errors", (double)ag.errors}, {"max_abs_diff", ag.max_abs}, {"max_rel_diff", ag.max_rel}});
  });
}

void run_gemv_accuracy(benchmark::State &state, const char *name) {
  guarded(state, [&] {
    const size_t M = state.range(0), K = state.range(1);
    if (M * K > ((size_t)1 << 28)) throw unsupported(std::string(name) + ": matrices beyond 2^28 elements are not multiplied on the host");
    const float alpha = 1.0f, beta = 0.0f;
    std::vector<float> hA(M * K), hx(K);
    fill_uniform01_f32(hA, flags().seed);
    fill_uniform01_f32(hx, flags().seed + 1);
    DeviceBuffer A(M * K * 2), x(K * 2), y(M * 4);
    upload_as_f16(hA, A);
    upload_as_f16(hx, x);
    PRINT_IF_ERROR(hipMemset(y.get(), 0, M * 4));
    EventPair ev;
    for (auto _ : state) {  // first: the 16-wide MFMA form on the fp16 operands
      ev.start();
      TCU_CHECK(tcu_gemv_f16_f32(A.get(), x.get(), y.get(), M, K, alpha, beta, TCU_VARIANT_MFMA_16N, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    std::vector<float> got(M);
    PRINT_IF_ERROR(hipMemcpy(got.data(), y.get(), M * 4, hipMemcpyDeviceToHost));
    // second: a single-precision product of the fp32 operands (the reference calls cublasSgemv)
    Agreement ag;
    for (size_t m = 0; m < M; m++) {
      float s = 0.0f;
      for (size_t k = 0; k < K; k++) s += hA[m * K + k] * hx[k];
      ag.add(alpha * s, got[m]);
    }
    state.counters.insert({{"M", (double)M}, {"N", (double)K}, {"errors", (double)ag.errors}, {"max_abs_diff", ag.max_abs}, {"max_rel_diff", ag.max_rel}});
  });
}

// ---------------------------------------------------------------------------------------
// the reference's CPU path, timed
// ---------------------------------------------------------------------------------------
static void cpu_reduce_range(const uint16_t *in, uint16_t *out, size_t seg0, size_t seg1, size_t S) {
  for (size_t j = seg0; j < seg1; j++) {
    float correct_segment_sum = 0;
    for (size_t i = 0; i < S; i++) correct_segment_sum += half_to_float(in[j * S + i]);
    out[j] = float_to_half(correct_segment_sum);
  }
}
static void cpu_scan_range(const uint16_t *in, uint16_t *out, size_t seg0, size_t seg1, size_t S) {
  for (size_t j = seg0; j < seg1; j++) {
    float running = 0;
    for (size_t i = 0; i < S; i++) {
      running += half_to_float(in[j * S + i]);
      out[j * S + i] = float_to_half(running);
    }
  }
}

void run_cpu_segmented(benchmark::State &state, bool scan, int threads) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), S = state.range(1), n = num_segments * S;
    if (threads <= 0) threads = (int)std::max(1u, std::thread::hardware_concurrency());
    std::vector<uint16_t> in(n), out(scan ? n : num_segments);
    {
      DeviceBuffer d(n * 2);
      TCU_CHECK(tcu_generate_f16(d.get(), n, 0, TCU_DIST_UNIFORM, 0, nullptr));  // seed 0: the CPU configuration
      PRINT_IF_ERROR(hipMemcpy(in.data(), d.get(), n * 2, hipMemcpyDeviceToHost));
    }
    for (auto _ : state) {
      const auto t0 = std::chrono::steady_clock::now();
      std::vector<std::thread> pool;
      for (int t = 0; t < threads; t++) {
        const size_t a = num_segments * t / threads, b = num_segments * (t + 1) / threads;
        if (scan)
          pool.emplace_back(cpu_scan_range, in.data(), out.data(), a, b, S);
        else
          pool.emplace_back(cpu_reduce_range, in.data(), out.data(), a, b, S);
      }
      for (auto &th : pool) th.join();
      state.SetIterationTime(std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
    }
    state.counters.insert({{"num_segments", (double)num_segments},
                           {"segment_size", (double)S},
                           {"num_elements", (double)n},
                           {"host_threads", (double)threads},
                           {"flops", {state.iterations() * 1.0 * n, benchmark::Counter::kAvgThreadsRate}}});
  });
}

}  // namespace harness
