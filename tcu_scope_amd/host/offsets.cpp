// Segments given by an offsets array: the hand-written counterparts of the reference's library baselines
// CUB_DEVICE_SEGMENTED_REDUCTION (cub::DeviceSegmentedReduce::Sum, src/reduction/seg_cub_device.cu:46-48) and
// THRUST_SEGMENTED_PREFIXSUM (src/prefixsum/seg_thrust.cu:46-47), on the same offsets and argument tuples.
#include "args.hpp"
#include "harness.hpp"

// ---- segmented reduction through an offsets array (the hand-written counterpart of the
// CUB_DEVICE_SEGMENTED_REDUCTION library baseline; same offsets, same argument tuples) ------------
static void TCU_OFFSETS_SEGMENTED_REDUCTION(benchmark::State &state) { harness::run_seg_reduce_offsets(state, true, "TCU_OFFSETS_SEGMENTED_REDUCTION"); }
// without the length hint: a whole wave per segment
static void TCU_OFFSETS_NOHINT_SEGMENTED_REDUCTION(benchmark::State &state) { harness::run_seg_reduce_offsets(state, false, "TCU_OFFSETS_NOHINT_SEGMENTED_REDUCTION"); }
BENCHMARK(TCU_OFFSETS_SEGMENTED_REDUCTION)->Apply(Tuning16_x_28)->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_REDUCTION)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_REDUCTION)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_REDUCTION)->SEG_4096_ARGS()->UseManualTime();
BENCHMARK(TCU_OFFSETS_NOHINT_SEGMENTED_REDUCTION)->Apply(Tuning16_x_28)->UseManualTime();
// inclusive prefix sums inside the segments of the same offsets array
static void TCU_OFFSETS_SEGMENTED_PREFIXSUM(benchmark::State &state) { harness::run_seg_scan_offsets(state, "TCU_OFFSETS_SEGMENTED_PREFIXSUM"); }
BENCHMARK(TCU_OFFSETS_SEGMENTED_PREFIXSUM)->Apply(Tuning16_x_28)->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_PREFIXSUM)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_PREFIXSUM)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(TCU_OFFSETS_SEGMENTED_PREFIXSUM)->SEG_2048_ARGS()->UseManualTime();
