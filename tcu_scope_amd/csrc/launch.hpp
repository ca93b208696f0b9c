// Kernel launch helper: launch(kernel, grid, block, stream, args...) enqueues `kernel`
// on the hipStream_t carried in `stream` (void*, NULL = default stream).
#ifndef TCU_LAUNCH_HPP
#define TCU_LAUNCH_HPP

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

namespace tcu {

// number of kernels this host thread has enqueued (lets callers tell "nothing was
// launched" from "a launch may have failed")
inline unsigned long &launch_count() {
  static thread_local unsigned long n = 0;
  return n;
}

// Events that the next launch of this host thread carries: the dispatch itself stamps them
// with the time the kernel starts and the time it ends (no separate packets on the stream).
struct LaunchEvents {
  hipEvent_t start = nullptr, stop = nullptr;
};
inline LaunchEvents &next_launch_events() {
  static thread_local LaunchEvents e;
  return e;
}

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), unsigned grid, unsigned block, void *stream, Args... args) {
  launch_count()++;
  LaunchEvents &ev = next_launch_events();
  if (ev.start || ev.stop) {
    hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, static_cast<hipStream_t>(stream), ev.start, ev.stop, 0, static_cast<KArgs>(args)...);
    ev = LaunchEvents{};
  } else {
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, static_cast<hipStream_t>(stream), static_cast<KArgs>(args)...);
  }
}

// Temporary device memory in stream order, from a memory pool of the library's own per device.
// The pool keeps what it has handed out once (release threshold at its maximum): the default
// pool gives unused memory back to the driver at every synchronisation, which turns the next
// request into a real allocation of a millisecond or more.  The block may be used by work
// enqueued on `stream` between stream_alloc and stream_free.  The pool is that of the stream's
// device (of the current device for the default stream).
// how many times the library has asked for temporary device memory (process-wide; tcu_temporary_allocations)
inline std::atomic<unsigned long> &stream_alloc_count() {
  static std::atomic<unsigned long> n{0};
  return n;
}
inline void *stream_alloc(size_t bytes, void *stream) {
  stream_alloc_count()++;
  constexpr int kMaxDevices = 64;
  static hipMemPool_t pools[kMaxDevices] = {};
  static std::mutex pools_mutex;
  int dev = 0;
  if (stream) {
    hipDevice_t of_stream = 0;
    if (hipStreamGetDevice(static_cast<hipStream_t>(stream), &of_stream) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    dev = (int)of_stream;
  } else if (hipGetDevice(&dev) != hipSuccess) {
    return nullptr;
  }
  if (dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> lock(pools_mutex);
  if (!pools[dev]) {
    hipMemPoolProps props = {};
    props.allocType = hipMemAllocationTypePinned;
    props.handleTypes = hipMemHandleTypeNone;
    props.location.type = hipMemLocationTypeDevice;
    props.location.id = dev;
    hipMemPool_t pool = nullptr;
    if (hipMemPoolCreate(&pool, &props) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    uint64_t keep = ~uint64_t{0};
    (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep);
    pools[dev] = pool;
  }
  void *p = nullptr;
  if (hipMallocFromPoolAsync(&p, bytes, pools[dev], static_cast<hipStream_t>(stream)) != hipSuccess) {
    (void)hipGetLastError();  // the caller reports the failure or does without; a later launch check must not see it
    return nullptr;
  }
  return p;
}
inline void stream_free(void *p, void *stream) { (void)hipFreeAsync(p, static_cast<hipStream_t>(stream)); }

}  // namespace tcu
#endif  // TCU_LAUNCH_HPP
