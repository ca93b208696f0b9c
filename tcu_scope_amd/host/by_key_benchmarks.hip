// Segments given by a key array, and the Thrust baselines.
//
// THRUST_SEGMENTED_REDUCTION / THRUST_SEGMENTED_PREFIXSUM (src/reduction/seg_thrust.cu:10-133,
// src/prefixsum/seg_thrust.cu:10-131: thrust::reduce_by_key / thrust::inclusive_scan_by_key over
// int keys = index / segment_size), THRUST_SEGMENTED2_PREFIXSUM (src/prefixsum/seg_thrust2.cu:
// one thrust::inclusive_scan call per segment), THRUST_FULL_REDUCTION / THRUST_FULL_PREFIXSUM
// (src/reduction/thrust.cu:11-89, src/prefixsum/thrust.cu:11-86) run rocThrust, the Thrust this
// GPU ships with.  TCU_BY_KEY_SEGMENTED_REDUCTION / TCU_BY_KEY_SEGMENTED_PREFIXSUM run the
// hand-written kernels behind tcu_seg_reduce_by_key_f16 / tcu_seg_scan_by_key_f16 on the same
// key arrays and argument tuples, and check their results against the fixed-size kernels'
// verifier.  Nothing of the product calls Thrust; the file only feeds the benchmark executable.
// Arithmetic of the baselines: fp16 in, fp32 accumulation, fp16 out (the reference adds in
// fp16), so they move the same bytes as the kernels they are compared with.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <thrust/execution_policy.h>
#include <thrust/iterator/transform_iterator.h>
#include <thrust/iterator/transform_output_iterator.h>
#include <thrust/reduce.h>
#include <thrust/scan.h>

#include "args.hpp"
#include "harness.hpp"

using harness::DeviceBuffer;
using harness::EventPair;

namespace {

struct HalfToFloat {
  __host__ __device__ float operator()(const __half &h) const { return __half2float(h); }
};
struct FloatToHalf {
  __host__ __device__ __half operator()(float v) const { return __float2half(v); }
};

__global__ void fill_keys(int *keys, size_t n, size_t segment_size) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) keys[i] = (int)(i / segment_size);
}

template <class Body>
void guarded(benchmark::State &state, Body body) {
  try {
    body();
  } catch (const std::exception &e) {
    state.SkipWithError(e.what());
  } catch (...) {
    state.SkipWithError("unknown exception");
  }
}

template <class Launch>
void timed_loop(benchmark::State &state, Launch launch) {
  EventPair ev;
  size_t it = 0;
  // one untimed call first, as the harness gives the hand-written kernels: the first launch out of a code object loads it
  launch(it++);
  PRINT_IF_ERROR(hipDeviceSynchronize());
  for (auto _ : state) {
    ev.start();
    launch(it++);
    const float ms = ev.stop_ms();
    state.PauseTiming();
    state.SetIterationTime(ms / 1000);
    state.ResumeTiming();
  }
}

void counters(benchmark::State &state, size_t num_segments, size_t segment_size, size_t num_elements, double bytes) {
  state.counters.insert({{"num_segments", (double)num_segments},
                         {"segment_size", (double)segment_size},
                         {"num_elements", (double)num_elements},
                         {"flops", {state.iterations() * 1.0 * num_elements, benchmark::Counter::kAvgThreadsRate}},
                         {"bytes_per_second", {state.iterations() * bytes, benchmark::Counter::kAvgThreadsRate}},
                         {"hbm_peak_fraction", {state.iterations() * bytes / 8e12, benchmark::Counter::kAvgThreadsRate}}});
}

// inputs of one segmented benchmark: two value arrays that alternate (none is served from the
// Infinity Cache) and the keys index / segment_size
struct KeyedInput {
  size_t num_segments, segment_size, n;
  int nin;
  DeviceBuffer in[2], keys;
  KeyedInput(benchmark::State &state)
      : num_segments(state.range(0)), segment_size(state.range(1)), n(num_segments * segment_size), nin(n <= ((size_t)1 << 29) ? 2 : 1),
        in{DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)}, keys(n * sizeof(int)) {
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    fill_keys<<<4096, 256>>>(static_cast<int *>(keys.get()), n, segment_size);
    PRINT_IF_ERROR(hipDeviceSynchronize());
  }
  const int *k() const { return static_cast<const int *>(keys.get()); }
  const __half *values(size_t it) const { return static_cast<const __half *>(in[it % nin].get()); }
};

void thrust_segmented_reduction(benchmark::State &state) {
  guarded(state, [&] {
    if ((size_t)state.range(0) * (size_t)state.range(1) >= ((size_t)1 << 31)) {
      state.SkipWithError("keys are 32-bit integers");
      return;
    }
    KeyedInput d(state);
    DeviceBuffer out(d.num_segments * 2), keys_out(d.num_segments * sizeof(int));
    timed_loop(state, [&](size_t it) {
      auto first = thrust::make_transform_iterator(d.values(it), HalfToFloat());
      thrust::reduce_by_key(thrust::device, d.k(), d.k() + d.n, first, static_cast<int *>(keys_out.get()), thrust::make_transform_output_iterator(static_cast<__half *>(out.get()), FloatToHalf()));
    });
    counters(state, d.num_segments, d.segment_size, d.n, 6.0 * d.n + 6.0 * d.num_segments);
  });
}

void thrust_segmented_prefixsum(benchmark::State &state) {
  guarded(state, [&] {
    if ((size_t)state.range(0) * (size_t)state.range(1) >= ((size_t)1 << 31)) {
      state.SkipWithError("keys are 32-bit integers");
      return;
    }
    KeyedInput d(state);
    DeviceBuffer out(d.n * 2);
    timed_loop(state, [&](size_t it) {
      auto first = thrust::make_transform_iterator(d.values(it), HalfToFloat());
      thrust::inclusive_scan_by_key(thrust::device, d.k(), d.k() + d.n, first, thrust::make_transform_output_iterator(static_cast<__half *>(out.get()), FloatToHalf()));
    });
    counters(state, d.num_segments, d.segment_size, d.n, 8.0 * d.n);
  });
}

// one library call per segment, as the reference's second Thrust baseline does
void thrust_segmented2_prefixsum(benchmark::State &state) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1), n = num_segments * segment_size;
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    DeviceBuffer out(n * 2);
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    timed_loop(state, [&](size_t it) {
      const __half *src = static_cast<const __half *>(in[it % nin].get());
      __half *dst = static_cast<__half *>(out.get());
      for (size_t s = 0; s < num_segments; s++) {
        auto first = thrust::make_transform_iterator(src + s * segment_size, HalfToFloat());
        thrust::inclusive_scan(thrust::device, first, first + segment_size, thrust::make_transform_output_iterator(dst + s * segment_size, FloatToHalf()));
      }
    });
    counters(state, num_segments, segment_size, n, 4.0 * n);
  });
}

void tcu_by_key_reduction(benchmark::State &state, const char *name) {
  guarded(state, [&] {
    if ((size_t)state.range(0) * (size_t)state.range(1) >= ((size_t)1 << 31)) {
      state.SkipWithError("keys are 32-bit integers");
      return;
    }
    KeyedInput d(state);
    DeviceBuffer out(d.n * 2), keys_out(d.n * sizeof(int)), num_runs(16);
    size_t ws_bytes = 0;
    TCU_CHECK(tcu_seg_reduce_by_key_f16(nullptr, nullptr, nullptr, nullptr, nullptr, d.n, 32, nullptr, &ws_bytes, nullptr));
    DeviceBuffer ws(ws_bytes);
    TCU_CHECK(tcu_seg_reduce_by_key_f16(d.k(), d.values(0), keys_out.get(), out.get(), num_runs.get(), d.n, 32, ws.get(), &ws_bytes, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    unsigned long long runs = 0;
    PRINT_IF_ERROR(hipMemcpy(&runs, num_runs.get(), sizeof(runs), hipMemcpyDeviceToHost));
    if (runs != d.num_segments) throw std::runtime_error(std::string(name) + ": wrong number of runs");
    if (harness::should_verify(d.n)) harness::verify_seg_reduce(d.values(0), out.get(), d.num_segments, d.segment_size, name);
    timed_loop(state, [&](size_t it) { TCU_CHECK(tcu_seg_reduce_by_key_f16(d.k(), d.values(it), keys_out.get(), out.get(), num_runs.get(), d.n, 32, ws.get(), &ws_bytes, nullptr)); });
    counters(state, d.num_segments, d.segment_size, d.n, 6.0 * d.n + 6.0 * d.num_segments);
  });
}

void tcu_by_key_prefixsum(benchmark::State &state, const char *name) {
  guarded(state, [&] {
    if ((size_t)state.range(0) * (size_t)state.range(1) >= ((size_t)1 << 31)) {
      state.SkipWithError("keys are 32-bit integers");
      return;
    }
    KeyedInput d(state);
    DeviceBuffer out(d.n * 2);
    size_t ws_bytes = 0;
    TCU_CHECK(tcu_seg_scan_by_key_f16(nullptr, nullptr, nullptr, d.n, 32, nullptr, &ws_bytes, nullptr));
    DeviceBuffer ws(ws_bytes);
    TCU_CHECK(tcu_seg_scan_by_key_f16(d.k(), d.values(0), out.get(), d.n, 32, ws.get(), &ws_bytes, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    if (harness::should_verify(d.n)) harness::verify_seg_scan(d.values(0), out.get(), d.num_segments, d.segment_size, name);
    timed_loop(state, [&](size_t it) { TCU_CHECK(tcu_seg_scan_by_key_f16(d.k(), d.values(it), out.get(), d.n, 32, ws.get(), &ws_bytes, nullptr)); });
    counters(state, d.num_segments, d.segment_size, d.n, 8.0 * d.n);
  });
}

}  // namespace

static void THRUST_FULL_REDUCTION(benchmark::State &state) {
  guarded(state, [&] {
    const size_t n = state.range(0);
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    float sum = 0.0f;  // thrust::reduce returns its result to the host, as in the reference
    timed_loop(state, [&](size_t it) {
      auto first = thrust::make_transform_iterator(static_cast<const __half *>(in[it % nin].get()), HalfToFloat());
      sum = thrust::reduce(thrust::device, first, first + n, 0.0f);
    });
    if (sum != sum && harness::flags().seed == ~0ull) throw std::runtime_error("unreachable");  // keeps the result alive
    counters(state, 1, n, n, 2.0 * n);
  });
}
BENCHMARK(THRUST_FULL_REDUCTION)->ARGS()->UseManualTime();

static void THRUST_FULL_PREFIXSUM(benchmark::State &state) {
  guarded(state, [&] {
    const size_t n = state.range(0);
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    DeviceBuffer out(n * 2);
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    timed_loop(state, [&](size_t it) {
      auto first = thrust::make_transform_iterator(static_cast<const __half *>(in[it % nin].get()), HalfToFloat());
      thrust::inclusive_scan(thrust::device, first, first + n, thrust::make_transform_output_iterator(static_cast<__half *>(out.get()), FloatToHalf()));
    });
    counters(state, 1, n, n, 4.0 * n);
  });
}
BENCHMARK(THRUST_FULL_PREFIXSUM)->ARGS()->UseManualTime();

#define ALL_SEGMENT_SIZES(NAME)                   \
  BENCHMARK(NAME)->SEG_16_ARGS()->UseManualTime();    \
  BENCHMARK(NAME)->SEG_32_ARGS()->UseManualTime();    \
  BENCHMARK(NAME)->SEG_64_ARGS()->UseManualTime();    \
  BENCHMARK(NAME)->SEG_128_ARGS()->UseManualTime();   \
  BENCHMARK(NAME)->SEG_256_ARGS()->UseManualTime();   \
  BENCHMARK(NAME)->SEG_512_ARGS()->UseManualTime();   \
  BENCHMARK(NAME)->SEG_1024_ARGS()->UseManualTime();  \
  BENCHMARK(NAME)->SEG_2048_ARGS()->UseManualTime();  \
  BENCHMARK(NAME)->SEG_4096_ARGS()->UseManualTime();  \
  BENCHMARK(NAME)->SEG_8192_ARGS()->UseManualTime();  \
  BENCHMARK(NAME)->SEG_16384_ARGS()->UseManualTime()
// the reference keeps its Thrust sweeps over growing segments commented out (RUN_THRUST_TUNE, src/reduction/seg_thrust.cu:139,
// src/prefixsum/seg_thrust.cu:130); its figure specifications still name them, so they are registered at the sizes of the other sweeps
#define ALL_SWEEPS(NAME)                                  \
  BENCHMARK(NAME)->Apply(Tuning16_x_14)->UseManualTime(); \
  BENCHMARK(NAME)->Apply(Tuning16_x_18)->UseManualTime(); \
  BENCHMARK(NAME)->Apply(Tuning16_x_22)->UseManualTime(); \
  BENCHMARK(NAME)->Apply(Tuning16_x_26)->UseManualTime(); \
  BENCHMARK(NAME)->Apply(Tuning16_x_28)->UseManualTime(); \
  BENCHMARK(NAME)->Apply(Tuning16_x_30)->UseManualTime()

static void THRUST_SEGMENTED_REDUCTION(benchmark::State &state) { thrust_segmented_reduction(state); }
static void THRUST_TUNE_SEGMENTED_REDUCTION(benchmark::State &state) { thrust_segmented_reduction(state); }
ALL_SEGMENT_SIZES(THRUST_SEGMENTED_REDUCTION);
ALL_SWEEPS(THRUST_TUNE_SEGMENTED_REDUCTION);

static void THRUST_SEGMENTED_PREFIXSUM(benchmark::State &state) { thrust_segmented_prefixsum(state); }
static void THRUST_TUNE_SEGMENTED_PREFIXSUM(benchmark::State &state) { thrust_segmented_prefixsum(state); }
ALL_SEGMENT_SIZES(THRUST_SEGMENTED_PREFIXSUM);
ALL_SWEEPS(THRUST_TUNE_SEGMENTED_PREFIXSUM);

static void THRUST_SEGMENTED2_PREFIXSUM(benchmark::State &state) { thrust_segmented2_prefixsum(state); }
static void THRUST_TUNE_SEGMENTED2_PREFIXSUM(benchmark::State &state) { thrust_segmented2_prefixsum(state); }
ALL_SEGMENT_SIZES(THRUST_SEGMENTED2_PREFIXSUM);
ALL_SWEEPS(THRUST_TUNE_SEGMENTED2_PREFIXSUM);

static void TCU_BY_KEY_SEGMENTED_REDUCTION(benchmark::State &state) { tcu_by_key_reduction(state, "TCU_BY_KEY_SEGMENTED_REDUCTION"); }
static void TCU_BY_KEY_TUNE_SEGMENTED_REDUCTION(benchmark::State &state) { tcu_by_key_reduction(state, "TCU_BY_KEY_TUNE_SEGMENTED_REDUCTION"); }
ALL_SEGMENT_SIZES(TCU_BY_KEY_SEGMENTED_REDUCTION);
ALL_SWEEPS(TCU_BY_KEY_TUNE_SEGMENTED_REDUCTION);

static void TCU_BY_KEY_SEGMENTED_PREFIXSUM(benchmark::State &state) { tcu_by_key_prefixsum(state, "TCU_BY_KEY_SEGMENTED_PREFIXSUM"); }
static void TCU_BY_KEY_TUNE_SEGMENTED_PREFIXSUM(benchmark::State &state) { tcu_by_key_prefixsum(state, "TCU_BY_KEY_TUNE_SEGMENTED_PREFIXSUM"); }
ALL_SEGMENT_SIZES(TCU_BY_KEY_SEGMENTED_PREFIXSUM);
ALL_SWEEPS(TCU_BY_KEY_TUNE_SEGMENTED_PREFIXSUM);
