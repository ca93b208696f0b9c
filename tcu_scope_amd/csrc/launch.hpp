// Kernel launch helper: launch(kernel, grid, block, stream, args...) enqueues `kernel`
// on the hipStream_t carried in `stream` (void*, NULL = default stream).
#ifndef TCU_LAUNCH_HPP
#define TCU_LAUNCH_HPP

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

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

// Temporary device memory in stream order (from the device's default memory pool: after the
// first use a request is served from the pool without a driver allocation).  The block may be
// used by work enqueued on `stream` between the two calls.
inline void *stream_alloc(size_t bytes, void *stream) {
  void *p = nullptr;
  if (hipMallocAsync(&p, bytes, static_cast<hipStream_t>(stream)) != hipSuccess) return nullptr;
  return p;
}
inline void stream_free(void *p, void *stream) { (void)hipFreeAsync(p, static_cast<hipStream_t>(stream)); }

}  // namespace tcu
#endif  // TCU_LAUNCH_HPP
