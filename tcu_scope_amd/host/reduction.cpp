// Reduction benchmarks under the reference's names and argument tuples
// (reference src/reduction/seg_wmma_*.cu, seg_cub_{warp,block}.cu, wmma_2kers*.cu,
// wmma_atomic.cu, wmma_cg.cu).  Template arguments keep their meaning:
// SEGMENTS_PER_WARP / tiles per wave, WARPS_PER_BLOCK, SEGMENT_SIZE.
#include "args.hpp"
#include "harness.hpp"

using harness::run_full_reduce;
using harness::run_seg_reduce;

// ---- MFMA families (the reference's WMMA kernels) -----------------------------------------
template <int SEGMENTS_PER_WARP, int WARPS_PER_BLOCK>
static void CUDA_WMMA_SEGMENTED_REDUCTION_16(benchmark::State &state) {
  if (state.range(1) != 16) {
    state.SkipWithError("segment size must be 16");
    return;
  }
  run_seg_reduce(state, TCU_VARIANT_MFMA_16, SEGMENTS_PER_WARP, WARPS_PER_BLOCK, "CUDA_WMMA_SEGMENTED_REDUCTION_16");
}
template <int SEGMENTS_PER_WARP, int WARPS_PER_BLOCK>
static void CUDA_WMMA_SEGMENTED_REDUCTION_256(benchmark::State &state) {
  if (state.range(1) != 256) {
    state.SkipWithError("segment size must be 256");
    return;
  }
  run_seg_reduce(state, TCU_VARIANT_MFMA_256, SEGMENTS_PER_WARP, WARPS_PER_BLOCK, "CUDA_WMMA_SEGMENTED_REDUCTION_256");
}
#define TCU_SEG_REDUCE_FAMILY(NAME, VARIANT)                                                           \
  template <int WARPS_PER_BLOCK>                                                                       \
  static void NAME(benchmark::State &state) {                                                          \
    run_seg_reduce(state, VARIANT, 0, WARPS_PER_BLOCK, #NAME);                                         \
  }
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_SEGMENTED_REDUCTION_16N, TCU_VARIANT_MFMA_16N)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_SEGMENTED_REDUCTION_16N_OPT, TCU_VARIANT_MFMA_16N)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_SEGMENTED_REDUCTION_16N_BLOCK, TCU_VARIANT_MFMA_16N_BLOCK)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_SEGMENTED_REDUCTION_256N, TCU_VARIANT_MFMA_256N)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_SEGMENTED_REDUCTION_256N_BLOCK, TCU_VARIANT_MFMA_256N_BLOCK)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_16N, TCU_VARIANT_MFMA_16N)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_16N_BLOCK, TCU_VARIANT_MFMA_16N_BLOCK)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N, TCU_VARIANT_MFMA_256N)
TCU_SEG_REDUCE_FAMILY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N_BLOCK, TCU_VARIANT_MFMA_256N_BLOCK)
// the fastest measured family and launch shape for every size
static void TCU_AUTO_SEGMENTED_REDUCTION(benchmark::State &state) { run_seg_reduce(state, TCU_VARIANT_AUTO, 0, 0, "TCU_AUTO_SEGMENTED_REDUCTION"); }

#define RUN_16(SPW)                                                                                    \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_16, SPW, 1)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_16, SPW, 2)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_16, SPW, 4)->SEG_16_ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_16, SPW, 8)->SEG_16_ARGS()->UseManualTime()
RUN_16(1);
RUN_16(2);
RUN_16(4);
RUN_16(8);
#define RUN_256(SPW)                                                                                   \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_256, SPW, 1)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_256, SPW, 2)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_256, SPW, 4)->SEG_256_ARGS()->UseManualTime();      \
  BENCHMARK_TEMPLATE(CUDA_WMMA_SEGMENTED_REDUCTION_256, SPW, 8)->SEG_256_ARGS()->UseManualTime()
RUN_256(1);
RUN_256(2);
RUN_256(4);
RUN_256(8);

// the reference's lists (src/reduction/seg_wmma_16n.cu:215-221, seg_wmma_16n_opt.cu:215-221, seg_wmma_16n_block.cu:229-235,
// seg_wmma_256n.cu:223-229, seg_wmma_256n_block.cu:242-248; tuning sweeps :206 / :212-214 of the same files), plus the
// sweeps over 2^28 elements that the measurements of this build are quoted on
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_REDUCTION_16N);
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_REDUCTION_16N_OPT);
RUN_WPB_SEG_16_TO_1024(CUDA_WMMA_SEGMENTED_REDUCTION_16N_BLOCK);
RUN_WPB_SEG_256_TO_16384(CUDA_WMMA_SEGMENTED_REDUCTION_256N);
RUN_WPB_SEG_256_TO_16384(CUDA_WMMA_SEGMENTED_REDUCTION_256N_BLOCK);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_16N, Tuning16_x_28);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_16N, Tuning16_x_30);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_16N_BLOCK, Tuning16_x_30);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N, Tuning256_x_22);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N, Tuning256_x_28);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N, Tuning256_x_30);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N_BLOCK, Tuning256_x_22);
RUN_WPB_APPLY(CUDA_WMMA_TUNE_SEGMENTED_REDUCTION_256N_BLOCK, Tuning256_x_30);
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->SEG_1024_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->SEG_4096_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->SEG_16384_ARGS()->UseManualTime();
BENCHMARK(TCU_AUTO_SEGMENTED_REDUCTION)->Apply(Tuning16_x_28)->UseManualTime();

// ---- wave / block collectives (the reference's cub::WarpReduce / cub::BlockReduce rows) -----
// THREADS_PER_BLOCK is the block size in threads of 64-lane waves; LOGICAL_WARP_SIZE is the
// segment size handled by a sub-wave, exactly as in the reference.
template <int THREADS_PER_BLOCK, int LOGICAL_WARP_SIZE>
static void CUB_WARP_SEGMENTED_REDUCTION(benchmark::State &state) {
  if (state.range(1) != LOGICAL_WARP_SIZE) {
    state.SkipWithError("segment size must equal the logical warp size");
    return;
  }
  // a block of 32 threads is half a wave here: it runs as one wave
  run_seg_reduce(state, TCU_VARIANT_WAVE_SHUFFLE, 0, THREADS_PER_BLOCK >= 64 ? THREADS_PER_BLOCK / 64 : 1, "CUB_WARP_SEGMENTED_REDUCTION");
}
enum { BLOCK_REDUCE_RAKING = 0 };
template <int THREADS_PER_BLOCK, int ITEMS_PER_THREAD, int ALGORITHM>
static void CUB_BLOCK_SEGMENTED_REDUCTION(benchmark::State &state) {
  if (state.range(1) != THREADS_PER_BLOCK * ITEMS_PER_THREAD) {
    state.SkipWithError("segment size must equal THREADS_PER_BLOCK * ITEMS_PER_THREAD");
    return;
  }
  // a lane takes 8 items per 128-bit load; ITEMS_PER_THREAD / 8 such loads stay in flight (at most 8); segments
  // below 512 halves lie inside one wave's tile and the block is a launch shape of the wave kernel
  const int tiles = ITEMS_PER_THREAD >= 64 ? 8 : ITEMS_PER_THREAD >= 32 ? 4 : ITEMS_PER_THREAD >= 16 ? 2 : 1;
  run_seg_reduce(state, TCU_VARIANT_BLOCK_LDS, tiles, THREADS_PER_BLOCK >= 64 ? THREADS_PER_BLOCK / 64 : 1, "CUB_BLOCK_SEGMENTED_REDUCTION");
}
RUN_CUB_WARP(CUB_WARP_SEGMENTED_REDUCTION);
RUN_CUB_BLOCK(CUB_BLOCK_SEGMENTED_REDUCTION, BLOCK_REDUCE_RAKING);
// The reference's twins on its unpatched copy of CUB (src/reduction/seg_cub_warp_original.cu, seg_cub_block_original.cu):
// the patch only changes how the library adds halves, which has no counterpart here, so the names run the same kernels.
template <int THREADS_PER_BLOCK, int LOGICAL_WARP_SIZE>
static void ORIGINAL_CUB_WARP_SEGMENTED_REDUCTION(benchmark::State &state) { CUB_WARP_SEGMENTED_REDUCTION<THREADS_PER_BLOCK, LOGICAL_WARP_SIZE>(state); }
template <int THREADS_PER_BLOCK, int ITEMS_PER_THREAD, int ALGORITHM>
static void ORIGINAL_CUB_BLOCK_SEGMENTED_REDUCTION(benchmark::State &state) { CUB_BLOCK_SEGMENTED_REDUCTION<THREADS_PER_BLOCK, ITEMS_PER_THREAD, ALGORITHM>(state); }
RUN_CUB_WARP(ORIGINAL_CUB_WARP_SEGMENTED_REDUCTION);
RUN_CUB_BLOCK(ORIGINAL_CUB_BLOCK_SEGMENTED_REDUCTION, BLOCK_REDUCE_RAKING);

// ---- full-array reduction --------------------------------------------------------------------
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_16(benchmark::State &state) {
  run_full_reduce(state, TCU_FULL_MULTI_KERNEL, SEGMENT_SIZE, WARPS_PER_BLOCK, "CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_16");
}
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_256(benchmark::State &state) {
  run_full_reduce(state, TCU_FULL_MULTI_KERNEL, SEGMENT_SIZE, WARPS_PER_BLOCK, "CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_256");
}
// single kernel with an atomic carry: the reference's atomic (block-sync / atomic-ballot) and
// cooperative-groups variants differ only in how a block agrees on its partial; here a block
// always combines through LDS, so the three names run the same kernel
// SEGMENT_SIZE is what a warp takes per step in the reference; a block of this build holds its whole partition in
// registers, at most 8 tiles (4096 halves) per wave: larger template arguments run with that partition
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_BLOCK_SYNC(benchmark::State &state) {
  run_full_reduce(state, TCU_FULL_SINGLE_PASS | TCU_FULL_MFMA, harness::single_pass_partition(SEGMENT_SIZE, WARPS_PER_BLOCK), WARPS_PER_BLOCK, "CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_BLOCK_SYNC");
}
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_ATOMIC_BALLOT(benchmark::State &state) {
  run_full_reduce(state, TCU_FULL_SINGLE_PASS | TCU_FULL_MFMA, harness::single_pass_partition(SEGMENT_SIZE, WARPS_PER_BLOCK), WARPS_PER_BLOCK, "CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_ATOMIC_BALLOT");
}
template <int SEGMENT_SIZE, int WARPS_PER_BLOCK>
static void CUDA_WMMA_FULL_REDUCTION_CG(benchmark::State &state) {
  run_full_reduce(state, TCU_FULL_SINGLE_PASS | TCU_FULL_MFMA, harness::single_pass_partition(SEGMENT_SIZE, WARPS_PER_BLOCK), WARPS_PER_BLOCK, "CUDA_WMMA_FULL_REDUCTION_CG");
}
static void TCU_AUTO_FULL_REDUCTION(benchmark::State &state) { run_full_reduce(state, TCU_FULL_AUTO, 0, 0, "TCU_AUTO_FULL_REDUCTION"); }

// the reference's lists: SEGMENT_SIZE 256 ... 16 * 256 for the two-kernel and atomic families
// (src/reduction/wmma_2kers.cu:189-193, wmma_atomic.cu:181-185), up to 1024 * 256 for the cooperative-groups one (wmma_cg.cu:184-195)
#define BENCHMARK_REDUCTION0(SEGMENT_SIZE, WARPS_PER_BLOCK)                                                                        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_16, SEGMENT_SIZE, WARPS_PER_BLOCK)->ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_2KERS_BASE_256, SEGMENT_SIZE, WARPS_PER_BLOCK)->ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_BLOCK_SYNC, SEGMENT_SIZE, WARPS_PER_BLOCK)->ARGS()->UseManualTime();        \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_ATOMIC_W_ATOMIC_BALLOT, SEGMENT_SIZE, WARPS_PER_BLOCK)->ARGS()->UseManualTime();     \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, WARPS_PER_BLOCK)->ARGS()->UseManualTime()
#define BENCHMARK_REDUCTION(SEGMENT_SIZE) \
  BENCHMARK_REDUCTION0(SEGMENT_SIZE, 1);  \
  BENCHMARK_REDUCTION0(SEGMENT_SIZE, 2);  \
  BENCHMARK_REDUCTION0(SEGMENT_SIZE, 4);  \
  BENCHMARK_REDUCTION0(SEGMENT_SIZE, 8);  \
  BENCHMARK_REDUCTION0(SEGMENT_SIZE, 16)
#define BENCHMARK_REDUCTION_CG(SEGMENT_SIZE)                                                          \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, 1)->ARGS()->UseManualTime();          \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, 2)->ARGS()->UseManualTime();          \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, 4)->ARGS()->UseManualTime();          \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, 8)->ARGS()->UseManualTime();          \
  BENCHMARK_TEMPLATE(CUDA_WMMA_FULL_REDUCTION_CG, SEGMENT_SIZE, 16)->ARGS()->UseManualTime()
BENCHMARK_REDUCTION(256);
BENCHMARK_REDUCTION(2 * 256);
BENCHMARK_REDUCTION(4 * 256);
BENCHMARK_REDUCTION(8 * 256);
BENCHMARK_REDUCTION(16 * 256);
BENCHMARK_REDUCTION_CG(32 * 256);
BENCHMARK_REDUCTION_CG(64 * 256);
BENCHMARK_REDUCTION_CG(128 * 256);
BENCHMARK_REDUCTION_CG(256 * 256);
BENCHMARK_REDUCTION_CG(512 * 256);
BENCHMARK_REDUCTION_CG(1024 * 256);
BENCHMARK(TCU_AUTO_FULL_REDUCTION)->ARGS()->UseManualTime();
