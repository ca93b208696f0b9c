// Argument spaces of the benchmarks: same tuples and argument names as the reference's
// generators (src/reduction/args.hpp:38-146, src/gemm/args.hpp, src/gemv/args.hpp), so that
// benchmark names and --benchmark_filter strings carry over.
#pragma once

#include <cstdint>

#include "minibench.hpp"

// The generators are plain functions of run-time parameters; the names the benchmark files
// use (ARGS, SEG_<S>_ARGS, Tuning<base>_x_<log2>) are thin wrappers that fix the parameters.
namespace argspace {
using Bench = benchmark::internal::Benchmark;

inline int64_t pow2(int64_t exponent) { return int64_t{1} << exponent; }
constexpr int64_t kSmallestLog2 = 12, kLargestLog2 = 30;  // element counts 2^12 .. 2^30

// {num_elements}
inline void element_counts(Bench *b) {
  b->ArgNames({"num_elements"});
  for (int64_t e = kSmallestLog2; e <= kLargestLog2; ++e) b->Args({pow2(e)});
}
// {num_segments, segment_size, num_elements} for one segment size over all element counts
inline void fixed_segment_size(Bench *b, int64_t segment_size) {
  b->ArgNames({"num_segments", "segment_size", "num_elements"});
  for (int64_t e = kSmallestLog2; e <= kLargestLog2; ++e) b->Args({pow2(e) / segment_size, segment_size, pow2(e)});
}
// {num_segments, segment_size, base_segment_size, max_elements_log2}: 2^log2_elements elements cut
// into ever longer segments, from the base size up to one segment
inline void growing_segments(Bench *b, int64_t base_segment_size, int64_t log2_elements) {
  b->ArgNames({"num_segments", "segment_size", "base_segment_size", "max_elements_log2"});
  for (int64_t segment_size = base_segment_size; segment_size <= pow2(log2_elements); segment_size *= 2)
    b->Args({pow2(log2_elements) / segment_size, segment_size, base_segment_size, log2_elements});
}
template <int64_t SEGMENT_SIZE>
void with_segment_size(Bench *b) {
  fixed_segment_size(b, SEGMENT_SIZE);
}
template <int64_t BASE, int64_t LOG2_ELEMENTS>
void with_growing_segments(Bench *b) {
  growing_segments(b, BASE, LOG2_ELEMENTS);
}
}  // namespace argspace

static inline int64_t two_power_i(int64_t p) { return argspace::pow2(p); }

#define ARGS() Apply(argspace::element_counts)
#define TCU_SEG_ARGS(S) Apply(argspace::with_segment_size<S>)
#define SEG_16_ARGS() TCU_SEG_ARGS(16)
#define SEG_32_ARGS() TCU_SEG_ARGS(32)
#define SEG_64_ARGS() TCU_SEG_ARGS(64)
#define SEG_128_ARGS() TCU_SEG_ARGS(128)
#define SEG_256_ARGS() TCU_SEG_ARGS(256)
#define SEG_512_ARGS() TCU_SEG_ARGS(512)
#define SEG_1024_ARGS() TCU_SEG_ARGS(1024)
#define SEG_2048_ARGS() TCU_SEG_ARGS(2048)
#define SEG_4096_ARGS() TCU_SEG_ARGS(4096)
#define SEG_8192_ARGS() TCU_SEG_ARGS(8192)
#define SEG_16384_ARGS() TCU_SEG_ARGS(16384)

// One registration per WARPS_PER_BLOCK of the reference's lists (1, 2, 4, 8, 16), and the reference's two lists of
// segment sizes: 16 ... 1024 for the *_16N* families (e.g. src/reduction/seg_wmma_16n.cu:215-221) and 256 ... 16384
// for the *_256N* families (src/reduction/seg_wmma_256n.cu:223-229)
#define RUN_WPB(NAME, ARGS_MACRO)                             \
  BENCHMARK_TEMPLATE(NAME, 1)->ARGS_MACRO()->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 2)->ARGS_MACRO()->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 4)->ARGS_MACRO()->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 8)->ARGS_MACRO()->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 16)->ARGS_MACRO()->UseManualTime()
#define RUN_WPB_APPLY(NAME, FN)                            \
  BENCHMARK_TEMPLATE(NAME, 1)->Apply(FN)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 2)->Apply(FN)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 4)->Apply(FN)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 8)->Apply(FN)->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 16)->Apply(FN)->UseManualTime()
#define RUN_WPB_SEG_16_TO_1024(NAME) \
  RUN_WPB(NAME, SEG_16_ARGS);        \
  RUN_WPB(NAME, SEG_32_ARGS);        \
  RUN_WPB(NAME, SEG_64_ARGS);        \
  RUN_WPB(NAME, SEG_128_ARGS);       \
  RUN_WPB(NAME, SEG_256_ARGS);       \
  RUN_WPB(NAME, SEG_512_ARGS);       \
  RUN_WPB(NAME, SEG_1024_ARGS)
#define RUN_WPB_SEG_256_TO_16384(NAME) \
  RUN_WPB(NAME, SEG_256_ARGS);         \
  RUN_WPB(NAME, SEG_512_ARGS);         \
  RUN_WPB(NAME, SEG_1024_ARGS);        \
  RUN_WPB(NAME, SEG_2048_ARGS);        \
  RUN_WPB(NAME, SEG_4096_ARGS);        \
  RUN_WPB(NAME, SEG_8192_ARGS);        \
  RUN_WPB(NAME, SEG_16384_ARGS)
// The reference's cub::Block* registrations: every (THREADS_PER_BLOCK, ITEMS_PER_THREAD) with 32 ... 1024 threads whose
// product is a segment size from 32 to 16384 (src/reduction/seg_cub_block.cu:145-288, src/prefixsum/seg_cub_block.cu:159-302)
#define RUN_CUB_BLOCK(NAME, ALG)                                                       \
  BENCHMARK_TEMPLATE(NAME, 32, 1, ALG)->SEG_32_ARGS()->UseManualTime();                \
  BENCHMARK_TEMPLATE(NAME, 32, 2, ALG)->SEG_64_ARGS()->UseManualTime();                \
  BENCHMARK_TEMPLATE(NAME, 64, 1, ALG)->SEG_64_ARGS()->UseManualTime();                \
  BENCHMARK_TEMPLATE(NAME, 32, 4, ALG)->SEG_128_ARGS()->UseManualTime();               \
  BENCHMARK_TEMPLATE(NAME, 64, 2, ALG)->SEG_128_ARGS()->UseManualTime();               \
  BENCHMARK_TEMPLATE(NAME, 128, 1, ALG)->SEG_128_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 32, 8, ALG)->SEG_256_ARGS()->UseManualTime();               \
  BENCHMARK_TEMPLATE(NAME, 64, 4, ALG)->SEG_256_ARGS()->UseManualTime();               \
  BENCHMARK_TEMPLATE(NAME, 128, 2, ALG)->SEG_256_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 256, 1, ALG)->SEG_256_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 32, 16, ALG)->SEG_512_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 64, 8, ALG)->SEG_512_ARGS()->UseManualTime();               \
  BENCHMARK_TEMPLATE(NAME, 128, 4, ALG)->SEG_512_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 256, 2, ALG)->SEG_512_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 512, 1, ALG)->SEG_512_ARGS()->UseManualTime();              \
  BENCHMARK_TEMPLATE(NAME, 32, 32, ALG)->SEG_1024_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 64, 16, ALG)->SEG_1024_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 128, 8, ALG)->SEG_1024_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 256, 4, ALG)->SEG_1024_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 512, 2, ALG)->SEG_1024_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 1024, 1, ALG)->SEG_1024_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 32, 64, ALG)->SEG_2048_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 64, 32, ALG)->SEG_2048_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 128, 16, ALG)->SEG_2048_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 256, 8, ALG)->SEG_2048_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 512, 4, ALG)->SEG_2048_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 1024, 2, ALG)->SEG_2048_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 32, 128, ALG)->SEG_4096_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 64, 64, ALG)->SEG_4096_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 128, 32, ALG)->SEG_4096_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 256, 16, ALG)->SEG_4096_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 512, 8, ALG)->SEG_4096_ARGS()->UseManualTime();             \
  BENCHMARK_TEMPLATE(NAME, 1024, 4, ALG)->SEG_4096_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 32, 256, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 64, 128, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 128, 64, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 256, 32, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 512, 16, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 1024, 8, ALG)->SEG_8192_ARGS()->UseManualTime();            \
  BENCHMARK_TEMPLATE(NAME, 32, 512, ALG)->SEG_16384_ARGS()->UseManualTime();           \
  BENCHMARK_TEMPLATE(NAME, 64, 256, ALG)->SEG_16384_ARGS()->UseManualTime();           \
  BENCHMARK_TEMPLATE(NAME, 128, 128, ALG)->SEG_16384_ARGS()->UseManualTime();          \
  BENCHMARK_TEMPLATE(NAME, 256, 64, ALG)->SEG_16384_ARGS()->UseManualTime();           \
  BENCHMARK_TEMPLATE(NAME, 512, 32, ALG)->SEG_16384_ARGS()->UseManualTime();           \
  BENCHMARK_TEMPLATE(NAME, 1024, 16, ALG)->SEG_16384_ARGS()->UseManualTime()
// cub::Warp*: 32 ... 1024 threads per block, logical warps of 16 and 32 (src/reduction/seg_cub_warp.cu:145-161)
#define RUN_CUB_WARP(NAME)                                        \
  BENCHMARK_TEMPLATE(NAME, 32, 16)->SEG_16_ARGS()->UseManualTime();   \
  BENCHMARK_TEMPLATE(NAME, 64, 16)->SEG_16_ARGS()->UseManualTime();   \
  BENCHMARK_TEMPLATE(NAME, 128, 16)->SEG_16_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 256, 16)->SEG_16_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 512, 16)->SEG_16_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 1024, 16)->SEG_16_ARGS()->UseManualTime(); \
  BENCHMARK_TEMPLATE(NAME, 32, 32)->SEG_32_ARGS()->UseManualTime();   \
  BENCHMARK_TEMPLATE(NAME, 64, 32)->SEG_32_ARGS()->UseManualTime();   \
  BENCHMARK_TEMPLATE(NAME, 128, 32)->SEG_32_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 256, 32)->SEG_32_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 512, 32)->SEG_32_ARGS()->UseManualTime();  \
  BENCHMARK_TEMPLATE(NAME, 1024, 32)->SEG_32_ARGS()->UseManualTime()

constexpr auto Tuning16_x_14 = argspace::with_growing_segments<16, 14>;
constexpr auto Tuning16_x_18 = argspace::with_growing_segments<16, 18>;
constexpr auto Tuning16_x_22 = argspace::with_growing_segments<16, 22>;
constexpr auto Tuning256_x_22 = argspace::with_growing_segments<256, 22>;
constexpr auto Tuning16_x_26 = argspace::with_growing_segments<16, 26>;
constexpr auto Tuning256_x_26 = argspace::with_growing_segments<256, 26>;
constexpr auto Tuning16_x_28 = argspace::with_growing_segments<16, 28>;
constexpr auto Tuning256_x_28 = argspace::with_growing_segments<256, 28>;
constexpr auto Tuning16_x_30 = argspace::with_growing_segments<16, 30>;
constexpr auto Tuning256_x_30 = argspace::with_growing_segments<256, 30>;

// GEMM: the reference's cubes (src/gemm/args.hpp:6-66): irregular steps up to 9216, then every 512 up to 28160
static inline void GemmArgs(benchmark::internal::Benchmark *b) {
  static const int64_t small[] = {16, 32, 48, 64, 96, 128, 192, 256, 512, 768, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192};
  for (int64_t s : small) b->Args({s, s, s});
  for (int64_t s = 9216; s <= 28160; s += 512) b->Args({s, s, s});
  b->ArgNames({"M", "N", "K"});
}
// GEMV: the reference's squares (src/gemv/args.hpp:6-65): irregular steps up to 1536, then every 512 from 2048 to 25600
static inline void GemvArgs(benchmark::internal::Benchmark *b) {
  static const int64_t small[] = {16, 32, 48, 64, 96, 128, 192, 256, 512, 1024, 1536};
  for (int64_t s : small) b->Args({s, s});
  for (int64_t s = 2048; s <= 25600; s += 512) b->Args({s, s});
  b->ArgNames({"M", "N"});
}
