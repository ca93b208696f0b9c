// Measurement aids that have no counterpart among the reference's benchmarks: the plain
// streaming kernels that give the machine's copy / read / write ceilings for a launch
// shape, and launch-shape sweeps of the segmented kernels (kernel family, 1 KiB tiles in
// flight per wave, waves per block) from which the AUTO launch shapes were chosen.
// Not part of `bench`: `make bench_probes` builds a second executable that has these names as well.
#include "../../include/tcu_scope_dev.h"
#include "args.hpp"
#include "harness.hpp"

using harness::DeviceBuffer;
using harness::EventPair;

namespace {

void run_stream_probe(benchmark::State &state, int mode, int tiles_per_wave, int waves_per_block) {
  try {
    const size_t num_elements = state.range(0), bytes = num_elements * 2;
    // two sources alternate and four destinations take turns, so that no launch is served from the memory-side
    // cache or overwrites lines an earlier launch left dirty in it
    const int nbuf = 2, ndst = 4;
    DeviceBuffer src[2] = {DeviceBuffer(bytes), DeviceBuffer(bytes)};
    DeviceBuffer dst[4] = {DeviceBuffer(bytes), DeviceBuffer(bytes), DeviceBuffer(bytes), DeviceBuffer(bytes)};
    for (int i = 0; i < nbuf; i++) harness::fill_input(src[i].get(), num_elements, harness::flags().seed + i);
    for (int i = 0; i < ndst; i++) TCU_CHECK(tcu_fill_f16(dst[i].get(), 0.0f, num_elements, nullptr));
    TCU_CHECK(tcu_stream_probe(dst[0].get(), src[0].get(), bytes, mode, tiles_per_wave, waves_per_block, nullptr));
    PRINT_IF_ERROR(hipDeviceSynchronize());
    EventPair ev;
    size_t it = 0;
    for (auto _ : state) {
      const size_t i = it++;
      ev.start();
      TCU_CHECK(tcu_stream_probe(dst[i % ndst].get(), src[i % nbuf].get(), bytes, mode, tiles_per_wave, waves_per_block, nullptr));
      const float ms = ev.stop_ms();
      state.PauseTiming();
      state.SetIterationTime(ms / 1000);
      state.ResumeTiming();
    }
    const double moved = mode == 0 ? 2.0 * bytes : (double)bytes;
    state.counters["num_elements"] = (double)num_elements;
    state.counters["tiles_per_wave"] = tiles_per_wave;
    state.counters["waves_per_block"] = waves_per_block;
    state.counters["bytes_per_second"] = benchmark::Counter(moved * state.iterations(), benchmark::Counter::kAvgThreadsRate);
    state.counters["hbm_peak_fraction"] = benchmark::Counter(moved * state.iterations() / 8e12, benchmark::Counter::kAvgThreadsRate);
  } catch (const std::exception &e) {
    state.SkipWithError(e.what());
  }
}

void StreamArgs(benchmark::internal::Benchmark *b) {
  for (int64_t l = 24; l <= 30; l += 2) b->Args({two_power_i(l)});
  b->ArgNames({"num_elements"});
}

}  // namespace

template <int TILES_PER_WAVE, int WAVES_PER_BLOCK>
static void TCU_STREAM_PROBE_COPY(benchmark::State &state) { run_stream_probe(state, 0, TILES_PER_WAVE, WAVES_PER_BLOCK); }
template <int TILES_PER_WAVE, int WAVES_PER_BLOCK>
static void TCU_STREAM_PROBE_READ(benchmark::State &state) { run_stream_probe(state, 1, TILES_PER_WAVE, WAVES_PER_BLOCK); }
template <int TILES_PER_WAVE, int WAVES_PER_BLOCK>
static void TCU_STREAM_PROBE_WRITE(benchmark::State &state) { run_stream_probe(state, 2, TILES_PER_WAVE, WAVES_PER_BLOCK); }

#define PROBE_SHAPES(NAME)                                          \
  BENCHMARK_TEMPLATE(NAME, 1, 1)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 2, 1)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 4, 1)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 1, 4)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 2, 4)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 4, 4)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 1, 16)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 2, 16)->Apply(StreamArgs)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 4, 16)->Apply(StreamArgs)->UseManualTime()
PROBE_SHAPES(TCU_STREAM_PROBE_COPY);
PROBE_SHAPES(TCU_STREAM_PROBE_READ);
PROBE_SHAPES(TCU_STREAM_PROBE_WRITE);

// ---- launch-shape sweeps at 2^28 elements, segment sizes 16 .. 2^28 ---------------------------
// VARIANT is a tcu_variant value (2 MFMA_16N, 3 MFMA_16N_BLOCK, 5 MFMA_256N, 6 MFMA_256N_BLOCK,
// 7 WAVE_SHUFFLE, 8 BLOCK_LDS); sizes a family does not support are reported as skipped.
template <int VARIANT, int TILES_PER_WAVE, int WAVES_PER_BLOCK>
static void TCU_SHAPE_SEGMENTED_REDUCTION(benchmark::State &state) {
  harness::run_seg_reduce(state, VARIANT, TILES_PER_WAVE, WAVES_PER_BLOCK, "TCU_SHAPE_SEGMENTED_REDUCTION");
}
template <int VARIANT, int TILES_PER_WAVE, int WAVES_PER_BLOCK>
static void TCU_SHAPE_SEGMENTED_PREFIXSUM(benchmark::State &state) {
  harness::run_seg_scan(state, VARIANT, TILES_PER_WAVE, WAVES_PER_BLOCK, false, "TCU_SHAPE_SEGMENTED_PREFIXSUM");
}
#define SHAPE_ONE(NAME, V, T, W) BENCHMARK_TEMPLATE(NAME, V, T, W)->Apply(Tuning16_x_28)->UseManualTime()
#define SHAPE_WAVES(NAME, V, T) \
  SHAPE_ONE(NAME, V, T, 1);     \
  SHAPE_ONE(NAME, V, T, 2);     \
  SHAPE_ONE(NAME, V, T, 4);     \
  SHAPE_ONE(NAME, V, T, 8);     \
  SHAPE_ONE(NAME, V, T, 16)
#define SHAPE_FAMILY(NAME, V) \
  SHAPE_WAVES(NAME, V, 1);    \
  SHAPE_WAVES(NAME, V, 2);    \
  SHAPE_WAVES(NAME, V, 4);    \
  SHAPE_WAVES(NAME, V, 8)
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_REDUCTION, TCU_VARIANT_MFMA_16N);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_REDUCTION, TCU_VARIANT_MFMA_16N_BLOCK);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_REDUCTION, TCU_VARIANT_MFMA_256N_BLOCK);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_REDUCTION, TCU_VARIANT_WAVE_SHUFFLE);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_REDUCTION, TCU_VARIANT_BLOCK_LDS);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_PREFIXSUM, TCU_VARIANT_MFMA_16N);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_PREFIXSUM, TCU_VARIANT_MFMA_16N_BLOCK);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_PREFIXSUM, TCU_VARIANT_MFMA_256N_BLOCK);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_PREFIXSUM, TCU_VARIANT_WAVE_SHUFFLE);
SHAPE_FAMILY(TCU_SHAPE_SEGMENTED_PREFIXSUM, TCU_VARIANT_BLOCK_LDS);
