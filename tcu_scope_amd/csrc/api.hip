// C ABI of libtcu_scope_amd.so (declared in include/tcu_scope.h): thin wrappers that
// validate, pick a kernel (dispatch.hpp) and report launch errors.
#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>

#include "dispatch.hpp"

// Partition descriptors of tcu_seg_scan_f16_noalloc: a ticket counter (64 words) and one 64-bit
// descriptor for each partition of 65536 halves: 256 bytes apart for up to 4096 partitions, closer
// together for more, 131072 partitions at most.  Every device the library's
// code is loaded on holds its own copy of the array, at its own address, until the process ends;
// `scratch` itself is only the host-side handle of the symbol, never a device address.
constexpr size_t kScratchMaxPartitions = 131072;
constexpr size_t kScratchWords = 64 + 2 * kScratchMaxPartitions;
static __device__ __align__(256) unsigned scratch[kScratchWords];

namespace {

// The address of `scratch` on the device the work will run on: the stream's device, or the current device for the
// default stream (the rule tcu::stream_alloc follows).  Resolved once per device (tcu_init does it for the device it
// selects; otherwise the first call that needs it); hipGetSymbolAddress answers for the current device, so a stream
// of another device makes that device current for the query and restores the caller's afterwards.
int scratch_on_device_of(const char *what, void *stream, unsigned **out) {
  constexpr int kMaxDevices = 64;
  static unsigned *address[kMaxDevices] = {};
  static std::mutex address_mutex;
  int current = 0;
  hipError_t e = hipGetDevice(&current);
  if (e != hipSuccess) return tcu::fail(TCU_ERR_RUNTIME, std::string(what) + ": hipGetDevice: " + hipGetErrorString(e));
  int dev = current;
  if (stream) {
    hipDevice_t of_stream = 0;
    e = hipStreamGetDevice(static_cast<hipStream_t>(stream), &of_stream);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return tcu::fail(TCU_ERR_RUNTIME, std::string(what) + ": hipStreamGetDevice: " + hipGetErrorString(e));
    }
    dev = (int)of_stream;
  }
  if (dev < 0 || dev >= kMaxDevices) return tcu::fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": device ordinal beyond what the library keeps scratch addresses for");
  std::lock_guard<std::mutex> lock(address_mutex);
  if (!address[dev]) {
    if (dev != current && (e = hipSetDevice(dev)) != hipSuccess) return tcu::fail(TCU_ERR_RUNTIME, std::string(what) + ": hipSetDevice: " + hipGetErrorString(e));
    unsigned *p = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
    if (dev != current) (void)hipSetDevice(current);
    if (e != hipSuccess || !p) {
      (void)hipGetLastError();
      return tcu::fail(TCU_ERR_RUNTIME, std::string(what) + ": hipGetSymbolAddress(scratch): " + hipGetErrorString(e));
    }
    address[dev] = p;
  }
  *out = address[dev];
  return TCU_OK;
}

struct DeviceState {
  bool initialised = false;
  int device = 0;
  int compute_units = 0;
  int wavefront = 0;
  int lds_bytes = 0;
  bool gfx950 = false;
};
DeviceState &state() {
  static DeviceState s;
  return s;
}

int runtime_error(const char *what, hipError_t e) { return tcu::fail(TCU_ERR_RUNTIME, std::string(what) + ": " + hipGetErrorString(e)); }

// Kernel launches are asynchronous; what can be caught here is a launch that the runtime
// rejected (bad configuration, no code object for the device).
int after_launch(const char *what, unsigned long launches_before, int rc) {
  // events armed by tcu_time_next_launch belong to this call: if it launched nothing (a rejected
  // argument, an empty input) they must not ride on some later, unrelated launch
  tcu::next_launch_events() = tcu::LaunchEvents{};
  if (rc != TCU_OK || tcu::launch_count() == launches_before) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return runtime_error(what, e);
  return TCU_OK;
}

}  // namespace

extern "C" {

int tcu_abi_version(void) { return TCU_SCOPE_ABI_VERSION; }

const char *tcu_last_error(void) { return tcu::last_error_string().c_str(); }

int tcu_init(int device_id) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess) return runtime_error("tcu_init: hipGetDeviceCount", e);
  if (count <= 0) return tcu::fail(TCU_ERR_RUNTIME, "tcu_init: no HIP device");
  if (device_id < 0 || device_id >= count) device_id = 0;  // as the reference does for --cuda_device_id
  e = hipSetDevice(device_id);
  if (e != hipSuccess) return runtime_error("tcu_init: hipSetDevice", e);
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, device_id);
  if (e != hipSuccess) return runtime_error("tcu_init: hipGetDeviceProperties", e);
  DeviceState &s = state();
  s.device = device_id;
  s.compute_units = prop.multiProcessorCount;
  s.wavefront = prop.warpSize;
  s.lds_bytes = (int)prop.sharedMemPerBlock;
  s.gfx950 = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
  s.initialised = true;
  if (s.compute_units > 0) tcu::options().compute_units = s.compute_units;
  if (!s.gfx950) return tcu::fail(TCU_ERR_UNSUPPORTED, std::string("tcu_init: this library is built for gfx950 only, device is ") + prop.gcnArchName);
  unsigned *scratch_address = nullptr;
  return scratch_on_device_of("tcu_init", nullptr, &scratch_address);
}

int tcu_device_info(int *compute_units, int *wavefront_size, int *lds_bytes, int *is_gfx950) {
  DeviceState &s = state();
  if (!s.initialised) {
    int rc = tcu_init(0);
    if (rc != TCU_OK && rc != TCU_ERR_UNSUPPORTED) return rc;
  }
  if (compute_units) *compute_units = s.compute_units;
  if (wavefront_size) *wavefront_size = s.wavefront;
  if (lds_bytes) *lds_bytes = s.lds_bytes;
  if (is_gfx950) *is_gfx950 = s.gfx950 ? 1 : 0;
  return TCU_OK;
}

int tcu_set_option(const char *name, int value) { return tcu::set_option(name, value); }

int tcu_seg_reduce_f16(const void *d_in, void *d_out, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_reduce_f16", before, tcu::seg_reduce_dispatch(d_in, d_out, num_segments, segment_size, variant, tiles_per_wave, waves_per_block, stream));
}

int tcu_seg_reduce_offsets_f16(const void *d_in, void *d_out, size_t num_segments, const void *d_begin_offsets, const void *d_end_offsets, int offset_bits, size_t expected_segment_size, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_reduce_offsets_f16", before, tcu::seg_reduce_offsets_dispatch(d_in, d_out, num_segments, d_begin_offsets, d_end_offsets, offset_bits, expected_segment_size, stream));
}

int tcu_seg_scan_f16(const void *d_in, void *d_out, void *d_totals, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_scan_f16", before, tcu::seg_scan_dispatch(d_in, d_out, d_totals, num_segments, segment_size, variant, tiles_per_wave, waves_per_block, stream));
}

int tcu_seg_scan_f16_noalloc(const void *d_in, void *d_out, void *d_totals, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream) {
  const char *what = "tcu_seg_scan_f16_noalloc";
  tcu::ScanScratch s;
  if (int rc = scratch_on_device_of(what, stream, &s.words)) return rc;
  s.capacity = kScratchWords;
  const unsigned long before = tcu::launch_count();
  return after_launch(what, before, tcu::seg_scan_dispatch(d_in, d_out, d_totals, num_segments, segment_size, variant, tiles_per_wave, waves_per_block, stream, what, s));
}

int tcu_seg_scan_offsets_f16(const void *d_in, void *d_out, size_t num_segments, const void *d_begin_offsets, const void *d_end_offsets, int offset_bits, size_t expected_segment_size, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_scan_offsets_f16", before, tcu::seg_scan_offsets_dispatch(d_in, d_out, num_segments, d_begin_offsets, d_end_offsets, offset_bits, expected_segment_size, stream));
}

int tcu_seg_scan_by_key_f16(const void *d_keys, const void *d_in, void *d_out, size_t n, int key_bits, void *d_workspace, size_t *workspace_bytes, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_scan_by_key_f16", before, tcu::seg_scan_by_key_dispatch(d_keys, d_in, d_out, n, key_bits, d_workspace, workspace_bytes, stream));
}

int tcu_seg_reduce_by_key_f16(const void *d_keys, const void *d_in, void *d_keys_out, void *d_out, void *d_num_runs, size_t n, int key_bits, void *d_workspace, size_t *workspace_bytes, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_seg_reduce_by_key_f16", before, tcu::seg_reduce_by_key_dispatch(d_keys, d_in, d_keys_out, d_out, d_num_runs, n, key_bits, d_workspace, workspace_bytes, stream));
}

int tcu_add_partial_sums_f16(void *d_out, const void *d_partial_sums, size_t num_segments, size_t segment_size, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_add_partial_sums_f16", before, tcu::add_partial_sums_dispatch(d_out, d_partial_sums, num_segments, segment_size, stream));
}

int tcu_full_reduce_f16(const void *d_in, void *d_out, size_t n, void *d_workspace, size_t *workspace_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_full_reduce_f16", before, tcu::full_reduce_dispatch(d_in, d_out, n, d_workspace, workspace_bytes, strategy, segment_size, waves_per_block, stream));
}

int tcu_full_scan_f16(const void *d_in, void *d_out, size_t n, void *d_workspace, size_t *workspace_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_full_scan_f16", before, tcu::full_scan_dispatch(d_in, d_out, n, d_workspace, workspace_bytes, strategy, segment_size, waves_per_block, stream));
}

int tcu_gemv_f16_f32(const void *d_A, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemv_f16_f32", before, tcu::gemv_dispatch(d_A, d_x, d_y, M, K, alpha, beta, variant, stream));
}

int tcu_gemm_f16_f32(const void *d_A, const void *d_B, const void *d_C, void *d_D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemm_f16_f32", before, tcu::gemm_dispatch(d_A, d_B, d_C, d_D, M, N, K, alpha, beta, variant, stream));
}

int tcu_gemv_f16_f16(const void *d_A, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemv_f16_f16", before, tcu::hgemv_dispatch(d_A, d_x, d_y, M, K, alpha, beta, variant, stream));
}

int tcu_gemv_col_major_f16_f32(const void *d_A, size_t lda, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemv_col_major_f16_f32", before, tcu::gemv_col_major_dispatch<float>("tcu_gemv_col_major_f16_f32", d_A, lda, d_x, d_y, M, K, alpha, beta, stream));
}

int tcu_gemv_col_major_f16_f16(const void *d_A, size_t lda, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemv_col_major_f16_f16", before, tcu::gemv_col_major_dispatch<tcu::half_t>("tcu_gemv_col_major_f16_f16", d_A, lda, d_x, d_y, M, K, alpha, beta, stream));
}

int tcu_gemm_f16_f16(const void *d_A, const void *d_B, const void *d_C, void *d_D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_gemm_f16_f16", before, tcu::hgemm_dispatch(d_A, d_B, d_C, d_D, M, N, K, alpha, beta, variant, stream));
}

int tcu_fill_f16(void *d, float value, size_t n, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_fill_f16", before, tcu::fill_dispatch(d, value, n, stream)); }

int tcu_convert_f32_to_f16(void *d_out, const void *d_in, size_t n, void *stream) { const unsigned long before = tcu::launch_count();
  return after_launch("tcu_convert_f32_to_f16", before, tcu::convert_dispatch(d_out, d_in, n, stream)); }

int tcu_generate_f16(void *d, size_t n, uint64_t seed, int dist, size_t first, void *stream) { const unsigned long before = tcu::launch_count();
  return after_launch("tcu_generate_f16", before, tcu::generate_dispatch(d, n, seed, dist, first, stream)); }

int tcu_stream_probe(void *d_dst, const void *d_src, size_t bytes, int mode, int tiles_per_wave, int waves_per_block, void *stream) {
  const unsigned long before = tcu::launch_count();
  return after_launch("tcu_stream_probe", before, tcu::stream_probe_dispatch(d_dst, d_src, bytes, mode, tiles_per_wave, waves_per_block, stream));
}

int tcu_time_next_launch(void *start_event, void *stop_event) {
  tcu::LaunchEvents &ev = tcu::next_launch_events();
  ev.start = static_cast<hipEvent_t>(start_event);
  ev.stop = static_cast<hipEvent_t>(stop_event);
  return TCU_OK;
}

unsigned long tcu_temporary_allocations(void) { return tcu::stream_alloc_count().load(); }

int tcu_lane_probe(void *d_out, size_t *out_words, void *stream) { const unsigned long before = tcu::launch_count();
  return after_launch("tcu_lane_probe", before, tcu::lane_probe_dispatch(d_out, out_words, stream)); }

}  // extern "C"
