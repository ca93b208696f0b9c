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

// Bytes of LDS that the next launch of this host thread asks for beyond what its kernel declares.  The kernel
// does not touch them: they cap how many of its blocks a compute unit holds at a time (160 KiB of LDS per unit),
// i.e. the bytes the unit has in flight, which copy-shaped kernels with blocks of several waves are sensitive to.
inline unsigned &next_launch_lds_pad() {
  static thread_local unsigned n = 0;
  return n;
}
// The pad a kernel can take: never more than the compute unit has left beside the kernel's own LDS; requests
// beyond 48 KiB need the kernel's limit raised once per device.  What was found out about a kernel is kept per host
// thread (the launch goes to the current device, as every launch of the library does).
inline unsigned usable_lds_pad(const void *kernel, unsigned pad) {
  struct Known { const void *kernel; int device; unsigned own, raised_to; };
  static thread_local Known known[32];
  static thread_local int n_known = 0;
  constexpr unsigned kLdsPerUnit = 160u * 1024u, kNeedsRaise = 48u * 1024u;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  Known *k = nullptr;
  for (int i = 0; i < n_known; i++)
    if (known[i].kernel == kernel && known[i].device == device) k = &known[i];
  if (!k) {
    hipFuncAttributes attr{};
    if (hipFuncGetAttributes(&attr, kernel) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    Known fresh{kernel, device, (unsigned)attr.sharedSizeBytes, 0u};
    if (n_known < 32) k = &(known[n_known++] = fresh);
    else k = &(known[0] = fresh);
  }
  if (k->own + 1024u >= kLdsPerUnit) return 0;
  if (pad > kLdsPerUnit - 1024u - k->own) pad = kLdsPerUnit - 1024u - k->own;
  if (pad > kNeedsRaise && pad > k->raised_to) {
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pad) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    k->raised_to = pad;
  }
  return pad;
}

template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), unsigned grid, unsigned block, void *stream, Args... args) {
  launch_count()++;
  LaunchEvents &ev = next_launch_events();
  unsigned pad = next_launch_lds_pad();
  next_launch_lds_pad() = 0;
  if (pad) pad = usable_lds_pad(reinterpret_cast<const void *>(kernel), pad);
  if (ev.start || ev.stop) {
    hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), pad, static_cast<hipStream_t>(stream), ev.start, ev.stop, 0, static_cast<KArgs>(args)...);
    ev = LaunchEvents{};
  } else {
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(block), pad, static_cast<hipStream_t>(stream), static_cast<KArgs>(args)...);
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
// A block that a stream gives back is kept for that stream's next request (up to kSpareBlocks blocks per process):
// work enqueued on one stream runs in order, so the next user of the block on the same stream cannot overtake the
// last one, and the pool's two calls (about 10 us of host time per request, which a caller that waits for every
// call sees in full) are skipped.  A request the spare does not satisfy goes to the pool; a returned block that
// finds no room goes back to it.
struct StreamBlocks {
  static constexpr int kSpareBlocks = 8, kOutstanding = 64;
  struct Block {
    void *p = nullptr, *stream = nullptr;
    size_t bytes = 0;
    int dev = 0;
  };
  std::mutex mutex;
  Block spare[kSpareBlocks], out[kOutstanding];
};
inline StreamBlocks &stream_blocks() {
  static StreamBlocks b;
  return b;
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
  if (bytes == 0) bytes = 1;
  StreamBlocks &sb = stream_blocks();
  {
    std::lock_guard<std::mutex> lock(sb.mutex);
    for (auto &s : sb.spare) {
      if (s.p && s.stream == stream && s.dev == dev && s.bytes >= bytes) {
        for (auto &o : sb.out) {
          if (!o.p) {  // remembered so that stream_free knows its size; no room to remember: the pool serves the request
            o = s;
            s = StreamBlocks::Block{};
            return o.p;
          }
        }
        break;
      }
    }
  }
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
  std::lock_guard<std::mutex> lock2(sb.mutex);
  for (auto &o : sb.out) {
    if (!o.p) {
      o.p = p;
      o.stream = stream;
      o.bytes = bytes;
      o.dev = dev;
      break;
    }
  }
  return p;
}
inline void stream_free(void *p, void *stream) {
  if (!p) return;
  StreamBlocks &sb = stream_blocks();
  void *evicted = nullptr, *evicted_stream = nullptr;
  bool kept = false;
  {
    std::lock_guard<std::mutex> lock(sb.mutex);
    for (auto &o : sb.out) {
      if (o.p != p) continue;
      StreamBlocks::Block b = o;
      o = StreamBlocks::Block{};
      if (b.stream != stream) break;  // given back on another stream than it was taken on: the pool orders that
      // this stream's spare, else a free place, else the place of the smallest block if that is smaller
      StreamBlocks::Block *at = nullptr;
      for (auto &s : sb.spare)
        if (s.p && s.stream == stream && s.dev == b.dev) at = &s;
      if (!at)
        for (auto &s : sb.spare)
          if (!s.p && !at) at = &s;
      if (!at) {
        at = &sb.spare[0];
        for (auto &s : sb.spare)
          if (s.bytes < at->bytes) at = &s;
      }
      if (at->p && at->bytes >= b.bytes) break;  // what is kept is at least as large
      evicted = at->p;
      evicted_stream = at->stream;
      *at = b;
      kept = true;
      break;
    }
  }
  if (evicted) {
    if (evicted_stream == stream) (void)hipFreeAsync(evicted, static_cast<hipStream_t>(stream));
    else (void)hipFree(evicted);  // that stream may be gone by now: not in its order, but after all work on the device
  }
  if (!kept) (void)hipFreeAsync(p, static_cast<hipStream_t>(stream));
}

}  // namespace tcu
#endif  // TCU_LAUNCH_HPP
