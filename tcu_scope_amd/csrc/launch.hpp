// Kernel launch helper: launch(kernel, grid, block, stream, args...) enqueues `kernel`
// on the hipStream_t carried in `stream` (void*, NULL = default stream).
#ifndef TCU_LAUNCH_HPP
#define TCU_LAUNCH_HPP

#include <hip/hip_runtime.h>

namespace tcu {

// number of kernels this host thread has enqueued (lets callers tell "nothing was
// launched" from "a launch may have failed")
inline unsigned long &launch_count() {
  static thread_local unsigned long n = 0;
  return n;
}

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), unsigned grid, unsigned block, void *stream, Args... args) {
  launch_count()++;
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, static_cast<hipStream_t>(stream), static_cast<KArgs>(args)...);
}

}  // namespace tcu
#endif  // TCU_LAUNCH_HPP
