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
