// Shared host-side pieces of the benchmark harnesses: flags, HIP error plumbing, device
// buffers, seeded inputs, verification against a CPU sum, and the timed loops.
// The shape of every harness follows the reference's (e.g. src/reduction/seg_wmma_16n.cu:12-178):
// validate arguments -> allocate -> fill -> [verify] -> timed loop with an event pair around
// each launch -> counters; any failure becomes state.SkipWithError.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/tcu_scope.h"
#include "minibench.hpp"

namespace harness {

struct Flags {
  int cuda_device_id = 0;            // --cuda_device_id (name kept from the reference, src/init/flags.cpp:4)
  std::string input = "uniform";     // --tcu_input=uniform|constant|grid   (constant = the reference's 0.001 fill)
  std::string verify = "auto";       // --tcu_verify=auto|all|none          (auto: up to 2^26 elements)
  uint64_t seed = 1;                 // --tcu_seed
  int out_buffers = 3;               // --tcu_out_buffers: output buffers the timed launches of the scan benchmarks take in turn
  std::vector<std::string> options;  // --tcu_option=<name>:<value>, handed to tcu_set_option after tcu_init
  int verbose = 0;                   // --v
  bool help = false;                 // --help / -h
};
Flags &flags();
// parses and removes the harness flags from argv (as the reference does before Google
// Benchmark sees the command line, src/init/flags.cpp:9-23)
void init_flags(int *argc, char **argv);
// selects the device (--cuda_device_id, clamped to 0 when absent) and prints what it found
bool init_device();

struct hip_error : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct unsupported : std::runtime_error {
  using std::runtime_error::runtime_error;
};
void check_hip(hipError_t e, const char *expr, const char *file, int line);
void check_tcu(int status, const char *expr);
#define PRINT_IF_ERROR(expr) ::harness::check_hip((expr), #expr, __FILE__, __LINE__)
#define TCU_CHECK(expr) ::harness::check_tcu((expr), #expr)

class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  explicit DeviceBuffer(size_t bytes);
  ~DeviceBuffer();
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  void *get() const { return p_; }
  size_t bytes() const { return n_; }

 private:
  void *p_ = nullptr;
  size_t n_ = 0;
};

class EventPair {
 public:
  EventPair();
  ~EventPair();
  void start();
  float stop_ms();  // records stop, waits for it, returns the elapsed time

 private:
  hipEvent_t a_, b_;
};

// host fp16 helpers (bit recipe of reference src/utils/fp16_conversion.hpp:91-114 for the
// widening direction; round-to-nearest-even for the narrowing one)
float half_to_float(uint16_t h);
uint16_t float_to_half(float f);

// fills d (n halves) according to --tcu_input
void fill_input(void *d, size_t n, uint64_t seed);
inline const char *input_dist_name() { return flags().input.c_str(); }
bool should_verify(size_t num_elements);

// |got - fp64 sum| <= 2 ulp_fp16(result) + 1e-3 * sqrt(segment size); throws on mismatch
void verify_seg_reduce(const void *d_in, const void *d_out, size_t num_segments, size_t segment_size, const char *what);
void verify_seg_scan(const void *d_in, const void *d_out, size_t num_segments, size_t segment_size, const char *what);

// timed loops; `expected_segment_size` = 0 accepts any size the variant supports
void run_seg_reduce(benchmark::State &state, int variant, int tiles_per_wave, int waves_per_block, const char *name);
// segmented reduction through an offsets array (offsets[j] = j * segment_size: the array the
// reference's CUB_DEVICE_SEGMENTED_REDUCTION harness builds, src/reduction/seg_cub_device.cu:18-22)
void run_seg_reduce_offsets(benchmark::State &state, bool pass_expected_size, const char *name);
void run_seg_scan_offsets(benchmark::State &state, const char *name);
void run_seg_scan(benchmark::State &state, int variant, int tiles_per_wave, int waves_per_block, bool with_totals, const char *name);
// Halves per block of the single-pass full-array kernels for the reference's template pair (SEGMENT_SIZE per warp
// and step, WARPS_PER_BLOCK): their product, capped at what a block of this build holds in registers (8 tiles of 512
// halves per wave); the reference's kernels loop over larger values, these do not need to
inline size_t single_pass_partition(size_t segment_size, int waves_per_block) {
  // a wave takes whole 512-half tiles: the reference's SEGMENT_SIZE = 256 instances run one tile per wave
  const size_t per_wave = segment_size < 512 ? 512 : segment_size;
  const size_t want = per_wave * (size_t)waves_per_block, most = (size_t)waves_per_block * 8 * 512;
  return want < most ? want : most;
}
void run_full_reduce(benchmark::State &state, int strategy, size_t segment_size, int waves_per_block, const char *name);
void run_full_scan(benchmark::State &state, int strategy, size_t segment_size, int waves_per_block, const char *name);
// half_out: y (GEMV) or C and D (GEMM) in fp16, the reference's H* benchmarks
// col_major: A column-major with lda = M (tcu_gemv_col_major_*; `variant` is not used)
void run_gemv(benchmark::State &state, int variant, const char *name, bool half_out = false, bool col_major = false);
void run_gemm(benchmark::State &state, int variant, const char *name, bool half_out = false);
// two computations of one product compared under the reference's agreement rule
// (src/gemm/accuracy.cu:259-268, src/gemv/accuracy.cu:314-323); counters: errors, max_abs_diff, max_rel_diff
void run_gemm_accuracy(benchmark::State &state, const char *name);
void run_gemv_accuracy(benchmark::State &state, const char *name);
// the reference's CPU verification loop (fp32 running sum per segment, fp16 result) timed on
// `threads` host threads; scan = prefix sums instead of totals
void run_cpu_segmented(benchmark::State &state, bool scan, int threads);

}  // namespace harness
