// CPU lane-level emulation of csrc/wave_ops.hpp (TEST INFRASTRUCTURE ONLY).
//
// Lets the kernel sources under tcu_scope_amd/csrc be compiled with a host compiler and
// executed lane by lane, so that indexing, lane-layout arithmetic and masks can be
// checked against the oracle without a GPU.  Every thread of a block is a ucontext
// fiber; cross-lane operations and barriers are rendezvous points.  The emulation is
// strict: a cross-lane operation that not every live lane of the wave reaches aborts.
//
// It encodes the same assumptions about gfx950 as the comment at the top of
// wave_ops.hpp (MFMA operand layouts, DPP source-lane rules); those assumptions are
// checked against the hardware by the GPU probe test.
#ifndef TCU_WAVE_OPS_HPP
#define TCU_WAVE_OPS_HPP

#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <ucontext.h>

#include <functional>
#include <vector>

#define __global__
#define __device__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define TCU_DEVICE inline

namespace emu {
struct Dim3 {
  unsigned x = 1, y = 1, z = 1;
};
inline Dim3 g_threadIdx, g_blockIdx, g_blockDim, g_gridDim;

struct Fiber {
  ucontext_t ctx;
  bool done = false;
};
// Fiber stacks are taken once and used again by every block of every launch: a fresh, zero-filled 256 KiB per thread
// and block was most of the emulator's run time (page faults).
constexpr size_t kFiberStackBytes = 256 * 1024;
inline char *fiber_stack(unsigned thread) {
  static std::vector<char *> pool;
  while (pool.size() <= thread) {
    char *p = static_cast<char *>(malloc(kFiberStackBytes));
    if (!p) {
      fprintf(stderr, "emu: out of memory for fiber stacks\n");
      abort();
    }
    pool.push_back(p);
  }
  return pool[thread];
}
struct WaveSync {
  int arrived = 0;
  unsigned gen = 0;
  int alive = 0;
  uint32_t slot[64][40];
};
struct BlockState {
  std::vector<Fiber> fibers;
  std::vector<WaveSync> waves;
  ucontext_t sched;
  int current = -1;
  int alive = 0;
  int bar_arrived = 0;
  unsigned bar_gen = 0;
  std::function<void()> body;
};
inline BlockState *g_blk = nullptr;

inline void die(const char *msg) {
  fprintf(stderr, "emu: %s (block %u thread %u)\n", msg, g_blockIdx.x, g_threadIdx.x);
  abort();
}
inline void yield() {
  BlockState *b = g_blk;
  swapcontext(&b->fibers[b->current].ctx, &b->sched);
}
inline void fiber_entry() {
  BlockState *b = g_blk;
  b->body();
  Fiber &f = b->fibers[b->current];
  f.done = true;
  b->alive--;
  WaveSync &w = b->waves[b->current / 64];
  w.alive--;
  if (w.arrived > 0) die("a lane exited while others of its wave wait at a cross-lane operation");
  if (b->bar_arrived > 0 && b->bar_arrived == b->alive) {  // s_barrier ignores terminated waves
    b->bar_arrived = 0;
    b->bar_gen++;
  }
  swapcontext(&f.ctx, &b->sched);
}
inline void wave_sync() {
  BlockState *b = g_blk;
  WaveSync &w = b->waves[b->current / 64];
  unsigned gen = w.gen;
  if (++w.arrived == w.alive) {
    w.arrived = 0;
    w.gen++;
  } else {
    while (w.gen == gen) yield();
  }
}
inline void block_sync() {
  BlockState *b = g_blk;
  unsigned gen = b->bar_gen;
  if (++b->bar_arrived == b->alive) {
    b->bar_arrived = 0;
    b->bar_gen++;
  } else {
    while (b->bar_gen == gen) yield();
  }
}
// Runs `body` once per thread of every block; blocks execute one after another in
// blockIdx order (which is also the order in which atomic tickets are handed out).
inline void launch(unsigned grid, unsigned block, std::function<void()> body) {
  if (block % 64 != 0) die("block size must be a multiple of 64");
  g_gridDim.x = grid;
  g_blockDim.x = block;
  for (unsigned bi = 0; bi < grid; bi++) {
    BlockState blk;
    g_blk = &blk;
    blk.body = body;
    blk.fibers.resize(block);
    blk.waves.resize(block / 64);
    for (auto &w : blk.waves) w.alive = 64;
    blk.alive = (int)block;
    g_blockIdx.x = bi;
    for (unsigned t = 0; t < block; t++) {
      Fiber &f = blk.fibers[t];
      getcontext(&f.ctx);
      f.ctx.uc_stack.ss_sp = fiber_stack(t);
      f.ctx.uc_stack.ss_size = kFiberStackBytes;
      f.ctx.uc_link = nullptr;
      makecontext(&f.ctx, (void (*)())fiber_entry, 0);
    }
    int remaining = (int)block;
    while (remaining > 0) {
      int progressed = 0;
      for (unsigned t = 0; t < block; t++) {
        Fiber &f = blk.fibers[t];
        if (f.done) continue;
        blk.current = (int)t;
        g_threadIdx.x = t;
        swapcontext(&blk.sched, &f.ctx);
        progressed++;
        if (f.done) remaining--;
      }
      if (!progressed) die("deadlock");
    }
    g_blk = nullptr;
  }
}
}  // namespace emu

#define threadIdx emu::g_threadIdx
#define blockIdx emu::g_blockIdx
#define blockDim emu::g_blockDim
#define gridDim emu::g_gridDim
inline void __syncthreads() { emu::block_sync(); }
inline int __float_as_int(float f) {
  int i;
  memcpy(&i, &f, 4);
  return i;
}
inline float __int_as_float(int i) {
  float f;
  memcpy(&f, &i, 4);
  return f;
}
inline unsigned __float_as_uint(float f) { return (unsigned)__float_as_int(f); }
inline float __uint_as_float(unsigned u) { return __int_as_float((int)u); }

namespace tcu {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr int DPP_QUAD_XOR1 = 0xB1;
constexpr int DPP_QUAD_XOR2 = 0x4E;
constexpr int DPP_ROW_SHR0 = 0x110;
constexpr int DPP_WAVE_SHR1 = 0x138;
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

inline int lane_id() { return (int)(threadIdx.x & 63u); }
inline int wave_in_block() { return (int)(threadIdx.x >> 6); }

inline emu::WaveSync &my_wave() { return emu::g_blk->waves[emu::g_blk->current / 64]; }

// source lane of a DPP control word for `lane`, or -1 when there is none
inline int dpp_source_lane(int ctrl, int lane) {
  const int row = lane & ~15, r = lane & 15;
  if (ctrl >= 0 && ctrl <= 0xFF) return (lane & ~3) | ((ctrl >> (2 * (lane & 3))) & 3);
  if (ctrl >= 0x101 && ctrl <= 0x10F) {  // row_shl
    int d = ctrl - 0x100;
    return r + d <= 15 ? row | (r + d) : -1;
  }
  if (ctrl >= 0x111 && ctrl <= 0x11F) {  // row_shr
    int d = ctrl - 0x110;
    return r >= d ? row | (r - d) : -1;
  }
  if (ctrl >= 0x121 && ctrl <= 0x12F) return row | ((r - (ctrl - 0x120)) & 15);  // row_ror
  if (ctrl == 0x130) return lane < 63 ? lane + 1 : -1;                           // wave_shl:1
  if (ctrl == 0x138) return lane > 0 ? lane - 1 : -1;                            // wave_shr:1
  if (ctrl == 0x140) return row | (15 - r);
  if (ctrl == 0x141) return (lane & ~7) | (7 - (lane & 7));
  if (ctrl == 0x142) return lane >= 16 ? (row - 16) | 15 : -1;  // row_bcast:15
  if (ctrl == 0x143) return lane >= 32 ? 31 : -1;               // row_bcast:31
  emu::die("unsupported DPP control");
  return -1;
}

template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND_CTRL = true>
inline unsigned dpp_u32(unsigned old, unsigned src) {
  auto &w = my_wave();
  const int lane = lane_id();
  w.slot[lane][0] = src;
  emu::wave_sync();
  unsigned res = old;
  const bool enabled = ((ROW_MASK >> (lane >> 4)) & 1) && ((BANK_MASK >> ((lane >> 2) & 3)) & 1);
  if (enabled) {
    int sl = dpp_source_lane(CTRL, lane);
    if (sl >= 0)
      res = w.slot[sl][0];
    else if (BOUND_CTRL)
      res = 0;
  }
  emu::wave_sync();
  return res;
}
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND_CTRL = true>
inline float dpp(float old, float src) {
  return __uint_as_float(dpp_u32<CTRL, ROW_MASK, BANK_MASK, BOUND_CTRL>(__float_as_uint(old), __float_as_uint(src)));
}

inline unsigned readlane_u32(unsigned x, int l) {
  auto &w = my_wave();
  w.slot[lane_id()][0] = x;
  w.slot[lane_id()][1] = (unsigned)l;
  emu::wave_sync();
  for (int k = 0; k < 64; k++)
    if (w.slot[k][1] != (unsigned)l) emu::die("readlane index is not wave-uniform");
  unsigned r = w.slot[l][0];
  emu::wave_sync();
  return r;
}
inline float readlane(float x, int l) { return __uint_as_float(readlane_u32(__float_as_uint(x), l)); }

inline unsigned long long ballot(bool pred) {
  auto &w = my_wave();
  w.slot[lane_id()][0] = pred ? 1u : 0u;
  emu::wave_sync();
  unsigned long long r = 0;
  for (int l = 0; l < 64; l++) r |= (unsigned long long)(w.slot[l][0] & 1u) << l;
  emu::wave_sync();
  return r;
}
inline void lane_swap(unsigned &a, unsigned &b, int width) {
  // a[upper half of each 2*width group] <-> b[lower half]
  auto &w = my_wave();
  const int lane = lane_id();
  w.slot[lane][0] = a;
  w.slot[lane][1] = b;
  emu::wave_sync();
  unsigned na = a, nb = b;
  if (lane & width)
    na = w.slot[lane - width][1];
  else
    nb = w.slot[lane + width][0];
  emu::wave_sync();
  a = na;
  b = nb;
}
inline void permlane16_swap(unsigned &a, unsigned &b) { lane_swap(a, b, 16); }
inline void permlane32_swap(unsigned &a, unsigned &b) { lane_swap(a, b, 32); }
inline float add_xor16(float x) {
  unsigned a = __float_as_uint(x), b = a;
  permlane16_swap(a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}
inline float add_xor32(float x) {
  unsigned a = __float_as_uint(x), b = a;
  permlane32_swap(a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}

inline float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) {
  auto &w = my_wave();
  const int lane = lane_id();
  memcpy(&w.slot[lane][0], &a, 16);
  memcpy(&w.slot[lane][4], &b, 16);
  emu::wave_sync();
  float4_t d = c;
  const int n = lane & 15;
  for (int i = 0; i < 4; i++) {
    const int m = 4 * (lane >> 4) + i;
    float acc = 0.0f;
    for (int kb = 0; kb < 4; kb++) {
      half8_t av, bv;
      memcpy(&av, &w.slot[16 * kb + m][0], 16);
      memcpy(&bv, &w.slot[16 * kb + n][4], 16);
      for (int e = 0; e < 8; e++) acc += (float)av[e] * (float)bv[e];
    }
    d[i] += acc;
  }
  emu::wave_sync();
  return d;
}
inline float16_t mfma_32x32x16(half8_t a, half8_t b, float16_t c) {
  auto &w = my_wave();
  const int lane = lane_id();
  memcpy(&w.slot[lane][0], &a, 16);
  memcpy(&w.slot[lane][4], &b, 16);
  emu::wave_sync();
  float16_t d = c;
  const int n = lane & 31;
  for (int i = 0; i < 16; i++) {
    const int m = 8 * (i / 4) + 4 * (lane >> 5) + (i % 4);
    float acc = 0.0f;
    for (int kb = 0; kb < 2; kb++) {
      half8_t av, bv;
      memcpy(&av, &w.slot[32 * kb + m][0], 16);
      memcpy(&bv, &w.slot[32 * kb + n][4], 16);
      for (int e = 0; e < 8; e++) acc += (float)av[e] * (float)bv[e];
    }
    d[i] += acc;
  }
  emu::wave_sync();
  return d;
}

inline float fdot2(half2_t a, half2_t b, float c) { return c + (float)a[0] * (float)b[0] + (float)a[1] * (float)b[1]; }
inline float sum8(half8_t v, float acc) {
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
  acc = fdot2(__builtin_shufflevector(v, v, 0, 1), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 2, 3), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 4, 5), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 6, 7), ones, acc);
  return acc;
}
inline half8_t splat8(float v) {
  half_t h = (half_t)v;
  half8_t r = {h, h, h, h, h, h, h, h};
  return r;
}
inline unsigned pack_f16x2(float lo, float hi) {
  half2_t h = {(half_t)lo, (half_t)hi};
  unsigned u;
  memcpy(&u, &h, 4);
  return u;
}
inline uint16_t f16_bits(float v) {
  half_t h = (half_t)v;
  uint16_t u;
  memcpy(&u, &h, 2);
  return u;
}
template <bool NT>
inline half8_t load_chunk(const half8_t *p) {
  return *p;
}
template <bool NT>
inline void store_chunk(uint4_t *p, uint4_t v) {
  *p = v;
}
constexpr int kStoreCached = 0, kStoreAlternate = 1, kStoreStream = 2;
template <int NT, int J>
constexpr bool kTileStoreNT = NT == kStoreStream || (NT == kStoreAlternate && J % 2 == 0);
template <int V>
struct Int {
  static constexpr int value = V;
};
template <int N, int J = 0, class F>
inline void static_for(F &&f) {
  if constexpr (J < N) {
    f(Int<J>{});
    static_for<N, J + 1>(f);
  }
}
inline void sched_fence() {}
// lanes run one after another here, so the transfer is a plain copy and nothing is in flight
using lds_addr_t = uintptr_t;
inline uintptr_t wave_uniform(uintptr_t x) { return x; }
inline lds_addr_t lds_address_of(const half_t *lds_pointer) { return reinterpret_cast<uintptr_t>(lds_pointer); }
inline void load_chunk_to_lds(const void *wave_base, uint32_t lane_byte_offset, lds_addr_t lds_base) {
  *reinterpret_cast<half8_t *>(lds_base + 16 * (uintptr_t)lane_id()) = *reinterpret_cast<const half8_t *>(static_cast<const char *>(wave_base) + lane_byte_offset);
}
template <int N>
inline void wait_vector_loads() {}
inline void block_barrier_lds_only() { emu::block_sync(); }
enum : int { kSchedMfma = 0x008, kSchedVmem = 0x010, kSchedVmemRead = 0x020, kSchedDsRead = 0x100, kSchedDsWrite = 0x200 };
template <int KIND, int COUNT>
inline void sched_group() {}
inline void wave_lds_fence() {
  emu::wave_sync();
}
inline unsigned atomic_add_u32(unsigned *p, unsigned v) {
  unsigned o = *p;
  *p = o + v;
  return o;
}
inline unsigned atomic_add_u32_acq_rel(unsigned *p, unsigned v) { return atomic_add_u32(p, v); }
inline float atomic_add_f32(float *p, float v) {
  float o = *p;
  *p = o + v;
  return o;
}
inline unsigned long long atomic_load_u64(const unsigned long long *p) { return *(const volatile unsigned long long *)p; }
inline void atomic_store_u64(unsigned long long *p, unsigned long long v) { *(volatile unsigned long long *)p = v; }
inline float atomic_load_f32(const float *p) { return *(const volatile float *)p; }
inline void device_fence_release() {}
inline void device_fence_acquire() {}
inline void spin_pause() { emu::yield(); }

}  // namespace tcu
#endif  // TCU_WAVE_OPS_HPP

// emulated launch.hpp
#ifndef TCU_LAUNCH_HPP
#define TCU_LAUNCH_HPP
namespace tcu {
inline unsigned &next_launch_lds_pad() {  // occupancy hint of the real launch: nothing to emulate
  static thread_local unsigned n = 0;
  return n;
}
template <typename... KArgs, typename... Args>
inline void launch(void (*kernel)(KArgs...), unsigned grid, unsigned block, void *, Args... args) {
  next_launch_lds_pad() = 0;
  emu::launch(grid, block, [=]() { kernel(static_cast<KArgs>(args)...); });
}
// launches run to completion before they return here, so plain host memory is "stream ordered"
inline void *stream_alloc(size_t bytes, void *) { return std::malloc(bytes ? bytes : 1); }
inline void stream_free(void *p, void *) { std::free(p); }
}  // namespace tcu
#endif
