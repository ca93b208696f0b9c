// Prefix-sum benchmarks under the reference's names and argument tuples
// (reference src/prefixsum/seg_wmma_*.cu, seg_cub_{warp,block}.cu, wmma_3kers*.cu, wmma_cg.cu,
// wmma_atomic.cu).
#include "args.hpp"
#include "harness.hpp"

using harness::run_full_scan;
using harness::run_seg_scan;

template <int SEGMENTS_PER_WARP, int WARPS_PER_BLOCK>
static void CUDA_WMMA_SEGMENTED_PREFIXSUM_16(benchmark::State &state) {
  if (state.range(1) != 16) {
    state.SkipWithError("segment size must be 16");
    return;
  }
  run_seg_scan(state, TCU_VARIANT_MFMA_16, SEGMENTS_PER_WARP, WARPS_PER_BLOCK, false, "CUDA_WMMA_SEGMENTED_PREFIXSUM_16");
}
template <int SEGMENTS_PER_WARP, int WARPS_PER_BLOCK>
static void CUDA_WMMA_SEGMENTED_PREFIXSUM_256(benchmark::State &state) {
  if (state.range(1) != 256) {
    state.SkipWithError("segment size must be 256");
    return;
  }
  run_seg_scan(state, TCU_VARIANT_MFMA_256, SEGMENTS_PER_WARP, WARPS_PER_BLOCK, false, "CUDA_WMMA_SEGMENTED_PREFIXSUM_256");
}
#define TCU_SEG_SCAN_FAMILY(NAME, VARIANT, TOTALS)                 \
  template <int WARPS_PER_BLOCK>                                   \
  static void NAME(benchmark::State &state) {                      \
    run_seg_scan(state, VARIANT, 0, WARPS_PER_BLOCK, TOTALS, #NAME); \
  }
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N, TCU_VARIANT_MFMA_16N, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N_OPT, TCU_VARIANT_MFMA_16N, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N_BLOCK, TCU_VARIANT_MFMA_16N_BLOCK, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_SEGMENTED_PREFIXSUM_256N, TCU_VARIANT_MFMA_256N, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_SEGMENTED_PREFIXSUM_256N_BLOCK, TCU_VARIANT_MFMA_256N_BLOCK, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_16N, TCU_VARIANT_MFMA_16N, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N, TCU_VARIANT_MFMA_256N, false)
TCU_SEG_SCAN_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N_BLOCK, TCU_VARIANT_MFMA_256N_BLOCK, false)
static void TCU_AUTO_SEGMENTED_PREFIXSUM(benchmark::State &state) { run_seg_scan(state, TCU_VARIANT_AUTO, 0, 0, false, "TCU_AUTO_SEGMENTED_PREFIXSUM"); }

#define RUN_16(SPW)                                                                                    \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_16, SPW, 1)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_16, SPW, 2)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_16, SPW, 4)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_16, SPW, 8)->SEG_16_ARGS()->UseManualTime()
RUN_16(1);
RUN_16(2);
RUN_16(4);
RUN_16(8);
#define RUN_256(SPW)                                                                                   \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_256, SPW, 1)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_256, SPW, 2)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_256, SPW, 4)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_PREFIXSUM_256, SPW, 8)->SEG_256_ARGS()->UseManualTime()
RUN_256(1);
RUN_256(2);
RUN_256(4);
RUN_256(8);
// the reference's lists (src/prefixsum/seg_wmma_16n.cu:217-223, seg_wmma_16n_opt.cu:217-223, seg_wmma_16n_block.cu:232-238,
// seg_wmma_256n.cu:216-222, seg_wmma_256n_block.cu:227-233; tuning sweeps :208 / :205-208 of the same files), plus the
// sweeps over 2^28 elements that the measurements of this build are quoted on
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N);
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N_OPT);
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_PREFIXSUM_16N_BLOCK);
RUN_WPB_SEG_256_TO_16384(CUDA_WMMA_SEGMENTED_PREFIXSUM_256N);
RUN_WPB_SEG_256_TO_16384(CUDA_WMMA_SEGMENTED_PREFIXSUM_256N_BLOCK);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_16N, Tuning16_x_28);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_16N, Tuning16_x_30);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N, Tuning256_x_22);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N, Tuning256_x_28);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N, Tuning256_x_30);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N_BLOCK, Tuning256_x_22);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_PREFIXSUM_256N_BLOCK, Tuning256_x_30);
BENCHMARK(TCU_AUTO_SEGMENTED_PREFIXSUM)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_PREFIXSUM)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_PREFIXSUM)->SEG_2048_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_PREFIXSUM)->SEG_16384_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_PREFIXSUM)->Apply(Tuning16_x_28)->UseManualTime();

template <int THREADS_PER_BLOCK, int LOGICAL_WARP_SIZE>
static void CUB_WARP_SEGMENTED_PREFIXSUM(benchmark::State &state) {
  if (state.range(1) != LOGICAL_WARP_SIZE) {
    state.SkipWithError("segment size must equal the logical warp size");
    return;
  }
  // a block of 32 threads is half a wave here: it runs as one wave
  run_seg_scan(state, TCU_VARIANT_WAVE_SHUFFLE, 0, THREADS_PER_BLOCK >= 64 ? THREADS_PER_BLOCK / 64 : 1, false, "CUB_WARP_SEGMENTED_PREFIXSUM");
}
enum { BLOCK_SCAN_RAKING = 0 };
template <int THREADS_PER_BLOCK, int ITEMS_PER_THREAD, int ALGORITHM>
static void CUB_BLOCK_SEGMENTED_PREFIXSUM(benchmark::State &state) {
  if (state.range(1) != THREADS_PER_BLOCK * ITEMS_PER_THREAD) {
    state.SkipWithError("segment size must equal THREADS_PER_BLOCK * ITEMS_PER_THREAD");
    return;
  }
  // as in the reduction: ITEMS_PER_THREAD / 8 loads in flight per lane; below 512 halves the block is a launch shape
  const int tiles = ITEMS_PER_THREAD >= 64 ? 8 : ITEMS_PER_THREAD >= 32 ? 4 : ITEMS_PER_THREAD >= 16 ? 2 : 1;
  run_seg_scan(state, TCU_VARIANT_BLOCK_LDS, tiles, THREADS_PER_BLOCK >= 64 ? THREADS_PER_BLOCK / 64 : 1, false, "CUB_BLOCK_SEGMENTED_PREFIXSUM");
}
RUN_CUB_WARP(CUB_WARP_SEGMENTED_PREFIXSUM);
RUN_CUB_BLOCK(CUB_BLOCK_SEGMENTED_PREFIXSUM, BLOCK_SCAN_RAKING);
// the reference's twins on its unpatched copy of CUB (src/prefixsum/seg_cub_warp_original.cu, seg_cub_block_original.cu)
template <int THREADS_PER_BLOCK, int LOGICAL_WARP_SIZE>
static void ORIGINAL_CUB_WARP_SEGMENTED_PREFIXSUM(benchmark::State &state) { CUB_WARP_SEGMENTED_PREFIXSUM<THREADS_PER_BLOCK, LOGICAL_WARP_SIZE>(state); }
template <int THREADS_PER_BLOCK, int ITEMS_PER_THREAD, int ALGORITHM>
static void ORIGINAL_CUB_BLOCK_SEGMENTED_PREFIXSUM(benchmark::State &state) { CUB_BLOCK_SEGMENTED_PREFIXSUM<THREADS_PER_BLOCK, ITEMS_PER_THREAD, ALGORITHM>(state); }
RUN_CUB_WARP(ORIGINAL_CUB_WARP_SEGMENTED_PREFIXSUM);
RUN_CUB_BLOCK(ORIGINAL_CUB_BLOCK_SEGMENTED_PREFIXSUM, BLOCK_SCAN_RAKING);

// ---- full-array prefix sum -----------------------------------------------------------------
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_PREFIXSUM_3KERS(benchmark::State &state) {
  run_full_scan(state, TCU_FULL_MULTI_KERNEL, SEGMENT_SIZE, WARPS_PER_BLOCK, "CUDA_WMMA_FULL_PREFIXSUM_3KERS");
}
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_PREFIXSUM_3KERS_BLOCK(benchmark::State &state) {
  run_full_scan(state, TCU_FULL_MULTI_KERNEL, SEGMENT_SIZE, WARPS_PER_BLOCK, "CUDA_WMMA_FULL_PREFIXSUM_3KERS_BLOCK");
}
// single pass (the reference's cooperative-groups and atomic-ballot kernels are disabled
// upstream; the decoupled look-back kernel takes their place)
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_PREFIXSUM_CG(benchmark::State &state) {
  run_full_scan(state, TCU_FULL_SINGLE_PASS | TCU_FULL_MFMA, harness::single_pass_partition(SEGMENT_SIZE, WARPS_PER_BLOCK), WARPS_PER_BLOCK, "CUDA_WMMA_FULL_PREFIXSUM_CG");
}
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_PREFIXSUM_ATOMIC_W_ATOMIC_BALLOT(benchmark::State &state) {
  run_full_scan(state, TCU_FULL_SINGLE_PASS | TCU_FULL_MFMA, harness::single_pass_partition(SEGMENT_SIZE, WARPS_PER_BLOCK), WARPS_PER_BLOCK, "CUDA_WMMA_FULL_PREFIXSUM_ATOMIC_W_ATOMIC_BALLOT");
}
static void TCU_AUTO_FULL_PREFIXSUM(benchmark::State &state) { run_full_scan(state, TCU_FULL_AUTO, 0, 0, "TCU_AUTO_FULL_PREFIXSUM"); }

// the reference's lists: SEGMENT_SIZE 256 ... 16 * 256 for the three-kernel family (src/prefixsum/wmma_3kers.cu:173-177),
// up to 256 * 256 for its block form (wmma_3kers_block.cu:175-183), up to 1024 * 256 for the single-kernel forms
// (wmma_cg.cu:196-207, wmma_atomic.cu:190-200)
#define BENCHMARK_FULL_SCAN(NAME, SEGMENT_SIZE)                                   \
  BENCHMARK_TEMPLATE(NAME, SEGMENT_SIZE, 1)->ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, SEGMENT_SIZE, 2)->ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, SEGMENT_SIZE, 4)->ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, SEGMENT_SIZE, 8)->ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, SEGMENT_SIZE, 16)->ARGS()->UseManualTime()
#define BENCHMARK_PRIFIXSUM(SEGMENT_SIZE)                                         \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_3KERS, SEGMENT_SIZE);              \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_3KERS_BLOCK, SEGMENT_SIZE);        \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_CG, SEGMENT_SIZE);                 \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_ATOMIC_W_ATOMIC_BALLOT, SEGMENT_SIZE)
#define BENCHMARK_PRIFIXSUM_LARGE(SEGMENT_SIZE)                                   \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_3KERS_BLOCK, SEGMENT_SIZE);        \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_CG, SEGMENT_SIZE);                 \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_ATOMIC_W_ATOMIC_BALLOT, SEGMENT_SIZE)
#define BENCHMARK_PRIFIXSUM_LARGEST(SEGMENT_SIZE)                                 \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_CG, SEGMENT_SIZE);                 \
  BENCHMARK_FULL_SCAN(CUDA_WMMA_FULL_PREFIXSUM_ATOMIC_W_ATOMIC_BALLOT, SEGMENT_SIZE)
BENCHMARK_PRIFIXSUM(256);
BENCHMARK_PRIFIXSUM(2 * 256);
BENCHMARK_PRIFIXSUM(4 * 256);
BENCHMARK_PRIFIXSUM(8 * 256);
BENCHMARK_PRIFIXSUM(16 * 256);
BENCHMARK_PRIFIXSUM_LARGE(32 * 256);
BENCHMARK_PRIFIXSUM_LARGE(64 * 256);
BENCHMARK_PRIFIXSUM_LARGE(128 * 256);
BENCHMARK_PRIFIXSUM_LARGE(256 * 256);
BENCHMARK_PRIFIXSUM_LARGEST(512 * 256);
BENCHMARK_PRIFIXSUM_LARGEST(1024 * 256);
BENCHMARK(TCU_AUTO_FULL_PREFIXSUM)->ARGS()->UseManualTime();
