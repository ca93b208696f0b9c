// Argument spaces of the benchmarks: same tuples and argument names as the reference's
// generators (src/reduction/args.hpp:38-146, src/gemm/args.hpp, src/gemv/args.hpp), so that
// benchmark names and --benchmark_filter strings carry over.
#pragma once

#include <cstdint>

#include "minibench.hpp"

static inline int64_t two_power_i(int64_t p) { return static_cast<int64_t>(1) << p; }

constexpr int64_t kMinElementsLog2 = 12, kMaxElementsLog2 = 30;

static inline void ArgsParams(benchmark::internal::Benchmark *b) {
  for (int64_t l = kMinElementsLog2; l <= kMaxElementsLog2; l++) b->Args({two_power_i(l)});
  b->ArgNames({"num_elements"});
}

template <int BASE_SEGMENT_SIZE>
static inline void ArgsParamsSegmented(benchmark::internal::Benchmark *b) {
  for (int64_t l = kMinElementsLog2; l <= kMaxElementsLog2; l++) {
    const int64_t num_elements = two_power_i(l);
    b->Args({num_elements / BASE_SEGMENT_SIZE, BASE_SEGMENT_SIZE, num_elements});
  }
  b->ArgNames({"num_segments", "segment_size", "num_elements"});
}

#define ARGS() Apply(ArgsParams)
#define SEG_16_ARGS() Apply(ArgsParamsSegmented<16>)
#define SEG_32_ARGS() Apply(ArgsParamsSegmented<32>)
#define SEG_64_ARGS() Apply(ArgsParamsSegmented<64>)
#define SEG_128_ARGS() Apply(ArgsParamsSegmented<128>)
#define SEG_256_ARGS() Apply(ArgsParamsSegmented<256>)
#define SEG_512_ARGS() Apply(ArgsParamsSegmented<512>)
#define SEG_1024_ARGS() Apply(ArgsParamsSegmented<1024>)
#define SEG_2048_ARGS() Apply(ArgsParamsSegmented<2048>)
#define SEG_4096_ARGS() Apply(ArgsParamsSegmented<4096>)
#define SEG_8192_ARGS() Apply(ArgsParamsSegmented<8192>)
#define SEG_16384_ARGS() Apply(ArgsParamsSegmented<16384>)

// fixed element count 2^MAX_ELEMENTS_LOG2, segment size swept from the base upwards
template <int BASE_SEGMENT_SIZE, int MAX_ELEMENTS_LOG2>
static inline void TuningArgs(benchmark::internal::Benchmark *b) {
  const int64_t num_elements = two_power_i(MAX_ELEMENTS_LOG2);
  for (int64_t num_segments = num_elements / BASE_SEGMENT_SIZE; num_segments >= 1; num_segments /= 2) {
    const int64_t segment_size = num_elements / num_segments;
    if (segment_size < BASE_SEGMENT_SIZE) continue;
    b->Args({num_segments, segment_size, BASE_SEGMENT_SIZE, MAX_ELEMENTS_LOG2});
  }
  b->ArgNames({"num_segments", "segment_size", "base_segment_size", "max_elements_log2"});
}
static inline void Tuning16_x_22(benchmark::internal::Benchmark *b) { TuningArgs<16, 22>(b); }
static inline void Tuning256_x_22(benchmark::internal::Benchmark *b) { TuningArgs<256, 22>(b); }
static inline void Tuning16_x_26(benchmark::internal::Benchmark *b) { TuningArgs<16, 26>(b); }
static inline void Tuning256_x_26(benchmark::internal::Benchmark *b) { TuningArgs<256, 26>(b); }
static inline void Tuning16_x_28(benchmark::internal::Benchmark *b) { TuningArgs<16, 28>(b); }
static inline void Tuning256_x_28(benchmark::internal::Benchmark *b) { TuningArgs<256, 28>(b); }
static inline void Tuning16_x_30(benchmark::internal::Benchmark *b) { TuningArgs<16, 30>(b); }
static inline void Tuning256_x_30(benchmark::internal::Benchmark *b) { TuningArgs<256, 30>(b); }

static inline void GemmArgs(benchmark::internal::Benchmark *b) {
  static const int64_t sizes[] = {16, 32, 48, 64, 96, 128, 192, 256, 512, 768, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192, 9216, 10240, 12288, 14336, 16384};
  for (int64_t s : sizes) b->Args({s, s, s});
  b->ArgNames({"M", "N", "K"});
}
static inline void GemvArgs(benchmark::internal::Benchmark *b) {
  static const int64_t sizes[] = {16, 32, 48, 64, 96, 128, 192, 256, 512, 1024, 1536, 2048, 2560, 3072, 3584, 4096, 5120, 6144, 7168, 8192, 9216, 10240, 12288, 14336, 16384, 20480, 24576};
  for (int64_t s : sizes) b->Args({s, s});
  b->ArgNames({"M", "N"});
}
